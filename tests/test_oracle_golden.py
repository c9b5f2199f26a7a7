"""The CPU oracle against the vectors the reference's own CPU code produced (tests/golden/*.npz)."""
import numpy as np
import pytest
import torch

from conftest import GOLDEN_DIR, load_golden
from oracle import ncn_oracle as O


def _weights(g, dtype):
    return [g[f"W{l}"].to(dtype) for l in range(g["meta"]["L"])]


def test_index_map_matches_reference_rows():
    rows = np.load(f"{GOLDEN_DIR}/index_map.npz")["rows"]
    assert rows.shape[0] > 1000
    for N, n, stage, b, o, idx in rows.tolist():
        assert O.group_pos_to_index(N, n, stage, b, o) == idx
    # the batched table agrees with the scalar form
    for N, n in ((256, 2), (48, 3), (128, 16), (32, 32)):
        for stage in range(0, 10):
            pos = O.stage_positions(N, n, stage)
            for b in (0, (N // n) - 1):
                for o in range(n):
                    assert int(pos[b, o]) == O.group_pos_to_index(N, n, stage, b, o)


@pytest.mark.parametrize("prec,tol", [("f64", 1e-12), ("f32", 2e-6)])
def test_forward_matches_reference(golden_case, prec, tol):
    name, g = golden_case
    dtype = torch.float64 if prec == "f64" else torch.float32
    mt = g["meta"]
    yi, ya = O.net_forward(g["x"].to(dtype), g["xa"].to(dtype), _weights(g, dtype), g["alpha"], mt["n"], mt["C"])
    assert O.rel_err(yi, g[f"ref_{prec}_yi"]) < tol
    assert O.rel_err(ya, g[f"ref_{prec}_ya"]) < tol


def test_literal_loops_match_reference_small():
    for name in ("small_n4_L3", "odd_n3_L3"):
        g = load_golden(name)
        mt = g["meta"]
        dt = torch.float64
        yi, ya = O.literal_net_forward(g["x"].to(dt), g["xa"].to(dt), _weights(g, dt), g["alpha"], mt["n"], mt["C"])
        assert O.rel_err(yi, g["ref_f64_yi"]) < 1e-12
        assert O.rel_err(ya, g["ref_f64_ya"]) < 1e-12


@pytest.mark.parametrize("which", ["closed_form_reversible", "closed_form_from_inputs", "autograd"])
def test_backward_matches_reference_f64(golden_case, which):
    name, g = golden_case
    mt = g["meta"]
    dt = torch.float64
    x, xa, Ws = g["x"].to(dt), g["xa"].to(dt), _weights(g, dt)
    dyi, dya = g["dyi"].to(dt), g["dya"].to(dt)
    a, n, C = g["alpha"], mt["n"], mt["C"]
    if which == "autograd":
        _, _, dx, dxa, dWs = O.net_autograd(x, xa, Ws, dyi, dya, a, n, C)
        tol = 1e-11
    elif which == "closed_form_from_inputs":
        dx, dxa, dWs = O.net_backward_from_inputs(x, xa, dyi, dya, Ws, a, n, C)
        tol = 1e-11
    else:
        yi, ya = O.net_forward(x, xa, Ws, a, n, C)
        xr, xar, dx, dxa, dWs = O.net_backward(yi, ya, dyi, dya, Ws, a, n, C)
        tol = 1e-9  # the inversion amplifies rounding by ~(1/m)^(n*L)
        assert O.rel_err(xr, x) < tol
        assert (xar - xa).abs().max().item() < tol
    assert O.rel_err(dx, g["ref_f64_dx"]) < tol
    assert O.rel_err(dxa, g["ref_f64_dxa"]) < tol
    for l in range(mt["L"]):
        assert O.rel_err(dWs[l], g[f"ref_f64_dW{l}"]) < tol, f"dW{l}"


def test_backward_matches_reference_f32(golden_case):
    name, g = golden_case
    mt = g["meta"]
    x, xa, Ws = g["x"], g["xa"], _weights(g, torch.float32)
    a, n, C = g["alpha"], mt["n"], mt["C"]
    # per-stage saved outputs (the reference's autograd node): fp32 oracle error vs the float64 reference
    # run must sit inside the 1e-5 parity bar
    _, _, dx, dxa, dWs = O.net_backward_checkpointed(x, xa, g["dyi"], g["dya"], Ws, a, n, C, save_every=1)
    assert O.rel_err(dx, g["ref_f64_dx"]) < 5e-6
    assert O.rel_err(dxa, g["ref_f64_dxa"]) < 5e-6
    for l in range(mt["L"]):
        assert O.rel_err(dWs[l], g[f"ref_f64_dW{l}"]) < 5e-6
    # whole-stack reversal from the final outputs only: rounding grows like (1/m)^(n*L), looser bar
    yi, ya = O.net_forward(x, xa, Ws, a, n, C)
    _, _, dx, dxa, dWs = O.net_backward(yi, ya, g["dyi"], g["dya"], Ws, a, n, C)
    amp = (1 / 0.9) ** (n * mt["L"])
    assert O.rel_err(dx, g["ref_f64_dx"]) < 1e-6 * max(amp, 10)
    assert O.rel_err(dxa, g["ref_f64_dxa"]) < 1e-6 * max(amp, 10)


def test_reference_invertible_variant_agrees():
    """RefInvTorchNaive (custom per-group Function) and RefTorchNaive (autograd) describe the same layer;
    the oracle reproduces both sets of vectors."""
    for name in ("small_n4_L3", "bench_like_n8_L5"):
        g = load_golden(name)
        for k in ("yi", "ya", "dx", "dxa", "dW0"):
            assert O.rel_err(g[f"inv_f64_{k}"], g[f"ref_f64_{k}"]) < 1e-10, (name, k)


@pytest.mark.parametrize("prec,tol", [("f64", 1e-13), ("f32", 1e-6)])
def test_single_step_inverse_matches_reference(prec, tol):
    z = load_golden("invert_step")
    dtype = torch.float64 if prec == "f64" else torch.float32
    yi, ya = z[f"{prec}_yi"], z[f"{prec}_ya"]
    Wi = z[f"{prec}_Wi"].reshape(1, 1, 1, 1, -1)
    Wj = z[f"{prec}_Wj"].reshape(1, 1, 1, 1, -1)
    for j in (0, 3, 7):
        x, a, _ = O._unstep(yi[None, None, None], ya[None, None, None], Wi, Wj, j, 0.9, 0.9, O.ACT_TANH)
        assert x.dtype == dtype
        assert O.rel_err(x[0, 0, 0], z[f"{prec}_xi_j{j}"]) < tol
        assert O.rel_err(a[0, 0, 0], z[f"{prec}_xa_j{j}"]) < tol
