"""The plain C restatement (oracle/ncn_oracle.c) against the vectors of the reference's own CPU code, against the
vectors of its Triton kernels, and against the Python oracle.  CPU only."""
import numpy as np
import pytest
import torch

from conftest import GOLDEN_CASES, load_golden, load_npz
from oracle import c_oracle as CO
from oracle import ncn_oracle as O


def _weights(g, dtype):
    return [g[f"W{l}"].to(dtype) for l in range(g["meta"]["L"])]


@pytest.mark.parametrize("name", GOLDEN_CASES)
@pytest.mark.parametrize("prec,tol", [("f64", 1e-12), ("f32", 3e-6)])
def test_forward_backward_match_reference_vectors(name, prec, tol):
    g = load_golden(name)
    mt = g["meta"]
    dt = torch.float64 if prec == "f64" else torch.float32
    yi, ya, dx, dxa, dWs = CO.net_forward_backward(g["x"].to(dt), g["xa"].to(dt), _weights(g, dt), g["dyi"].to(dt),
                                                   g["dya"].to(dt), g["alpha"], mt["n"], mt["C"])
    # the reversible backward amplifies rounding by (1/m)^n per stage; float64 leaves room, float32 is held to the
    # forward only plus gradients at the amplified bar
    assert O.rel_err(yi, g[f"ref_{prec}_yi"]) < tol
    assert O.rel_err(ya, g[f"ref_{prec}_ya"]) < tol
    gtol = tol * (1 / 0.9) ** mt["n"] * (10 if prec == "f64" else 1)
    assert O.rel_err(dx, g[f"ref_{prec}_dx"]) < gtol
    assert O.rel_err(dxa, g[f"ref_{prec}_dxa"]) < gtol
    for l in range(mt["L"]):
        assert O.rel_err(dWs[l], g[f"ref_{prec}_dW{l}"]) < gtol, l


def test_inverse_round_trip_and_reference_inverse_vectors():
    g = load_golden("small_n4_L3")
    mt = g["meta"]
    dt = torch.float64
    Ws = _weights(g, dt)
    yi, ya = CO.net_forward(g["x"].to(dt), g["xa"].to(dt), Ws, g["alpha"], mt["n"], mt["C"])
    assert O.rel_err(yi, g["inv_f64_yi"]) < 1e-12          # RefInvTorchNaive's forward
    x, xa = CO.net_inverse(yi, ya, Ws, g["alpha"], mt["n"], mt["C"])
    assert O.rel_err(x, g["x"].to(dt)) < 1e-11 and O.rel_err(xa, g["xa"].to(dt)) < 1e-11


@pytest.mark.parametrize("act,code", [("tanh", 0), ("leaky-relu", 3), ("none", -1)])
def test_activations_match_triton_vectors(act, code):
    g = load_npz("triton_activations")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    for stage in (0, 1, 3):
        tag = f"{act}_l{stage}_"
        t = lambda k: torch.from_numpy(np.ascontiguousarray(g[tag + k]))
        yi, ya = CO.stage_forward(t("x"), t("xa"), t("W"), float(g["alpha"]), n, C, stage, activation=code)
        assert O.rel_err(yi, t("yi")) < 3e-6 and O.rel_err(ya, t("ya")) < 3e-6
        _, _, dx, dxa, dW = CO.stage_backward(yi, ya, t("dyi"), t("dya"), t("W"), float(g["alpha"]), n, C, stage,
                                              activation=code)
        assert O.rel_err(dx, t("dx")) < 3e-6 and O.rel_err(dxa, t("dxa")) < 3e-6
        assert O.rel_err(dW, t("dW0")) < 3e-6


def test_headline_tile_matches_triton_vectors():
    g = load_npz("triton_headline_tile")
    batch, N, E, C, n, L = (int(v) for v in g["meta"])
    t = lambda k: torch.from_numpy(np.ascontiguousarray(g[k])).double()
    yi, ya, dx, dxa, dWs = CO.net_forward_backward(t("x"), t("xa"), [t(f"W{l}") for l in range(L)], t("dyi"), t("dya"),
                                                   float(g["alpha"]), n, C)
    for got, key in ((yi, "yi"), (ya, "ya"), (dx, "dx"), (dxa, "dxa")):
        assert O.rel_err(got, t(key)) < 3e-6, key
    for l in range(L):
        assert O.rel_err(dWs[l], t(f"dW{l}")) < 3e-6


@pytest.mark.parametrize("case", [
    (2, 32, 16, 2, 4, 0, 3, 0), (3, 48, 30, 3, 3, 1, 2, 3), (1, 256, 32, 1, 2, 0, 8, 0), (2, 64, 128, 4, 16, 2, 3, 2),
    (2, 24, 12, 2, 1, 0, 2, -1), (2, 40, 6, 2, 5, 1000003, 2, 1), (1, 64, 256, 2, 32, 3, 1, 0),
    (2, 64, 16, 16, 2, 0, 5, 0), (2, 64, 8, 8, 16, 1, 2, 0),      # one feature per head
], ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d_a%d" % c)
def test_matches_python_oracle(case):
    batch, N, E, C, n, first, L, act = case
    d = torch.float64
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=21, xa_zero=False)
    ref = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.85, n, C, activation=act,
                         first_stage=first)
    got = CO.net_forward_backward(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.85, n, C,
                                  activation=act, first_stage=first)
    tol = 1e-12 * (1 / 0.9) ** n
    for k in range(4):
        assert O.rel_err(got[k], ref[k]) < tol, k
    for l in range(L):
        assert O.rel_err(got[4][l], ref[4][l]) < tol, l
    # dya = NULL is dya = 0
    a = CO.net_forward_backward(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), None, 0.85, n, C, activation=act,
                                first_stage=first)
    b = CO.net_forward_backward(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), torch.zeros_like(dy).to(d), 0.85, n,
                                C, activation=act, first_stage=first)
    assert torch.equal(a[2], b[2]) and torch.equal(a[4][0], b[4][0])


def test_refuses_what_it_cannot_hold():
    x = torch.zeros(1, 130, 4)
    with pytest.raises(ValueError):
        CO.stage_forward(x, x, torch.zeros(8), 0.9, 65, 1, 0)      # more rows per group than the C arrays hold
    with pytest.raises(ValueError):
        CO.stage_forward(torch.zeros(1, 4, 6), torch.zeros(1, 4, 6), torch.zeros(12), 0.9, 3, 1, 0)   # N % n != 0


@pytest.mark.parametrize("case", [(3, 32, 16, 2, 4, 2, 0), (2, 30, 12, 3, 5, 1, 3), (4, 64, 32, 1, 16, 2, 2), (2, 24, 8, 2, 3, 2, -1)],
                         ids=lambda c: "b%d_N%d_E%d_C%d_n%d_L%d_a%d" % c)
def test_tables_and_lengths_match_python_oracle(case):
    batch, N, E, C, n, L, act = case
    d = torch.float64
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=8, xa_zero=False)
    gen = torch.Generator().manual_seed(N)
    tables = [torch.randperm(N, generator=gen) for _ in range(L)]
    for lens in (None, [N] * batch, [int(v) for v in torch.randint(0, N + 1, (batch,), generator=gen)]):
        ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, tables,
                                     lens, activation=act)
        got = CO.net_forward_backward(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C,
                                      activation=act, tables=tables, ctx_len=lens)
        tol = 1e-12 * (1 / 0.9) ** n
        for k in range(4):
            assert O.rel_err(got[k], ref[k]) < tol, (lens, k)
        for l in range(L):
            assert O.rel_err(got[4][l], ref[4][l]) < tol, (lens, l)
    # the stride map as a table is the closed form, bit for bit
    st = [O.stride_group_table(N, n, l) for l in range(L)]
    a = CO.net_forward_backward(x, xa, Ws, dy, dya, 0.9, n, C, activation=act)
    b = CO.net_forward_backward(x, xa, Ws, dy, dya, 0.9, n, C, activation=act, tables=st)
    assert all(torch.equal(p, q) for p, q in zip(a[:4], b[:4]))


def test_tables_and_lengths_match_triton_vectors():
    """The older Triton kernels' outputs (tests/golden/triton_tables_lengths.npz): whole-group lengths forward and
    backward on the live rows, the cut group's live rows forward."""
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    alpha = float(g["alpha"])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    codes = {"tanh": 0, "leaky-relu": 3}
    for k in range(int(g["n_whole"])):
        tag = f"whole{k}_"
        table = t(g["table_" + str(g[tag + "table"])])
        live = t(g[tag + "live"])[:, :, None].expand(batch, N, E)
        if not bool(live.any()):
            continue
        x, W = t(g[tag + "x"]), t(g[tag + "W"])
        got = CO.net_forward_backward(x, torch.zeros_like(x), [W], t(g[tag + "dyi"]), t(g[tag + "dya"]), alpha, n, C,
                                      activation=codes[str(g[tag + "act"])], tables=[table], ctx_len=t(g[tag + "ctx_len"]))
        for got_k, key in zip(got[:4], ("yi", "ya", "dx", "dxa")):
            assert O.rel_err(got_k[live], t(g[tag + key])[live]) < 3e-6, (k, key)
        assert O.rel_err(got[4][0], t(g[tag + "dW0"])) < 3e-6, k
    for k in range(int(g["n_cut"])):
        tag = f"cut{k}_"
        table = t(g["table_" + str(g[tag + "table"])])
        check = t(g[tag + "check"])[:, :, None].expand(batch, N, E)
        x, W = t(g[tag + "x"]), t(g[tag + "W"])
        yi, ya = CO.stage_forward(x, torch.zeros_like(x), W, alpha, n, C, 0, table=table, ctx_len=t(g[tag + "ctx_len"]))
        assert O.rel_err(yi[check], t(g[tag + "yi"])[check]) < 3e-6 and O.rel_err(ya[check], t(g[tag + "ya"])[check]) < 3e-6


def test_reversal_without_kept_outputs_is_the_same_in_float64():
    d = torch.float64
    x, xa, Ws, dy, dya = O.make_inputs(2, 64, 32, 4, 4, seed=2, xa_zero=False)
    args = (x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, 4, 2)
    a = CO.net_forward_backward(*args)
    b = CO.net_forward_backward(*args, keep_outputs=False)
    for p, q in zip(a[:4], b[:4]):
        assert O.rel_err(q, p) < 1e-12
    for p, q in zip(a[4], b[4]):
        assert O.rel_err(q, p) < 1e-12


def test_cut_group_backward_matches_triton_vectors():
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    codes = {"tanh": 0, "leaky-relu": 3}
    for k in range(int(g["n_cutbwd"])):
        tag = f"cutbwd{k}_"
        live = t(g[tag + "live"])[:, :, None].expand(batch, N, E)
        x, W = t(g[tag + "x"]), t(g[tag + "W"])
        got = CO.net_forward_backward(x, torch.zeros_like(x), [W], t(g[tag + "dyi"]), t(g[tag + "dya"]), float(g["alpha"]),
                                      n, C, activation=codes[str(g[tag + "act"])], tables=[t(g[tag + "table"])],
                                      ctx_len=t(g[tag + "ctx_len"]))
        for got_k, key in zip(got[:4], ("yi", "ya", "dx", "dxa")):
            assert O.rel_err(got_k[live], t(g[tag + key])[live]) < 3e-6, (k, key)
        assert O.rel_err(got[4][0], t(g[tag + "dW0"])) < 3e-6, k
