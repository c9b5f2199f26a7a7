"""The HIP path against what the reference's Triton kernels produced under Triton's CPU interpreter
(tests/golden/triton_*.npz): activations by name, the stack class of the reference's bench script, grouping by a
table and context lengths.  Calls go through the module surfaces that mirror the reference's
(ncn_cuda_amd.ncn_triton, ncn_cuda_amd.chunk_linear), i.e. through autograd and the C ABI."""
import numpy as np
import pytest
import torch

from conftest import load_npz
from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-5   # float32, max |diff| / max |ref|


@pytest.fixture(scope="module")
def surfaces():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import chunk_linear, ncn_triton
    return ncn_triton, chunk_linear


def _g(a, grad=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.requires_grad_() if grad else t


@pytest.mark.parametrize("act", ["tanh", "leaky-relu", "none"])
@pytest.mark.parametrize("stage", [0, 1, 3])
def test_activation_by_name(surfaces, act, stage):
    T, _ = surfaces
    g = load_npz("triton_activations")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    tag = f"{act}_l{stage}_"
    x, xa, W = _g(g[tag + "x"], True), _g(g[tag + "xa"], True), _g(g[tag + "W"], True)
    yi, ya = T.fused_ncn_triton(x, xa, W, float(g["alpha"]), act, C, n, stage)
    torch.autograd.backward([yi, ya], [_g(g[tag + "dyi"]), _g(g[tag + "dya"])])
    for got, key in ((yi, "yi"), (ya, "ya"), (x.grad, "dx"), (xa.grad, "dxa"), (W.grad, "dW0")):
        assert O.rel_err(got.detach().cpu(), torch.from_numpy(g[tag + key])) < TOL, key


def test_leaky_relu_stack_class(surfaces):
    T, _ = surfaces
    g = load_npz("triton_activations")
    batch, N, E, C, n, L = (int(v) for v in g["net_meta"])
    Ws = [_g(g[f"net_W{l}"], True) for l in range(L)]
    x, xa = _g(g["net_x"], True), _g(g["net_xa"], True)
    net = T.NCNNetTestTriton(float(g["alpha"]), "leaky-relu", n, C, L, Ws)
    yi, ya = net(x, xa)
    torch.autograd.backward([yi, ya], [_g(g["net_dyi"]), _g(g["net_dya"])])
    for got, key in ((yi, "net_yi"), (ya, "net_ya"), (x.grad, "net_dx"), (xa.grad, "net_dxa")):
        assert O.rel_err(got.detach().cpu(), torch.from_numpy(g[key])) < TOL, key
    for l in range(L):
        assert O.rel_err(Ws[l].grad.cpu(), torch.from_numpy(g[f"net_dW{l}"])) < TOL, l


@pytest.mark.parametrize("k", list(range(18)))
def test_tables_and_whole_group_lengths(surfaces, k):
    _, CL = surfaces
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    tag = f"whole{k}_"
    live = torch.from_numpy(g[tag + "live"])[:, :, None].expand(batch, N, E)
    if not bool(live.any()):
        pytest.skip("no live row in this case")
    table = _g(g["table_" + str(g[tag + "table"])])
    ctx = _g(g[tag + "ctx_len"])
    x, W = _g(g[tag + "x"], True), _g(g[tag + "W"], True)
    xa = torch.zeros_like(x).requires_grad_()          # the reference's forward starts xa from zeros
    yi, ya = CL.fused_chunk_linear_ncn(x, xa, W, table, ctx, float(g["alpha"]), str(g[tag + "act"]), C, n, 0)
    torch.autograd.backward([yi, ya], [_g(g[tag + "dyi"]), _g(g[tag + "dya"])])
    for got, key in ((yi, "yi"), (ya, "ya"), (x.grad, "dx"), (xa.grad, "dxa")):
        assert O.rel_err(got.detach().cpu()[live], torch.from_numpy(g[tag + key])[live]) < TOL, key
    # dead rows carry no upstream gradient in the fixture and pass through here: dW is the live rows' alone
    assert O.rel_err(W.grad.cpu(), torch.from_numpy(g[tag + "dW0"])) < TOL


@pytest.mark.parametrize("k", list(range(6)))
def test_cut_group_forward_live_rows(surfaces, k):
    _, CL = surfaces
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    tag = f"cut{k}_"
    check = torch.from_numpy(g[tag + "check"])[:, :, None].expand(batch, N, E)
    table = _g(g["table_" + str(g[tag + "table"])])
    x, W = _g(g[tag + "x"]), _g(g[tag + "W"])
    yi, ya = CL.fused_chunk_linear_ncn(x, torch.zeros_like(x), W, table, _g(g[tag + "ctx_len"]), float(g["alpha"]),
                                       "tanh", C, n, 0)
    assert O.rel_err(yi.cpu()[check], torch.from_numpy(g[tag + "yi"])[check]) < TOL
    assert O.rel_err(ya.cpu()[check], torch.from_numpy(g[tag + "ya"])[check]) < TOL


@pytest.mark.parametrize("storage", ["f32", "bf16"])
def test_headline_tile_stack(surfaces, storage):
    """The tile of the headline shape (groups of 16 rows, heads of 32 features, 3 stages) against the reference's
    Triton stack class; bfloat16 storage with float32 arithmetic at 2e-2."""
    T, _ = surfaces
    g = load_npz("triton_headline_tile")
    batch, N, E, C, n, L = (int(v) for v in g["meta"])
    dt, tol = (torch.float32, TOL) if storage == "f32" else (torch.bfloat16, 2e-2)
    Ws = [_g(g[f"W{l}"]).to(dt).requires_grad_() for l in range(L)]
    x, xa = _g(g["x"]).to(dt).requires_grad_(), _g(g["xa"]).to(dt).requires_grad_()
    yi, ya = T.NCNNetTestTriton(float(g["alpha"]), "tanh", n, C, L, Ws)(x, xa)
    torch.autograd.backward([yi, ya], [_g(g["dyi"]).to(dt), _g(g["dya"]).to(dt)])
    for got, key in ((yi, "yi"), (ya, "ya"), (x.grad, "dx"), (xa.grad, "dxa")):
        assert O.rel_err(got.detach().float().cpu(), torch.from_numpy(g[key])) < tol, key
    for l in range(L):
        assert O.rel_err(Ws[l].grad.float().cpu(), torch.from_numpy(g[f"dW{l}"])) < tol, l


@pytest.mark.parametrize("k", list(range(6)))
def test_cut_group_forward_and_backward(surfaces, k):
    """A length that cuts a group, both directions, against the reference's kernels (fixtures with position 0 among
    the dead rows): forward, dx, dxa on the live rows and dW."""
    _, CL = surfaces
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    tag = f"cutbwd{k}_"
    live = torch.from_numpy(g[tag + "live"])[:, :, None].expand(batch, N, E)
    x, W = _g(g[tag + "x"], True), _g(g[tag + "W"], True)
    xa = torch.zeros_like(x).requires_grad_()
    yi, ya = CL.fused_chunk_linear_ncn(x, xa, W, _g(g[tag + "table"]), _g(g[tag + "ctx_len"]), float(g["alpha"]),
                                       str(g[tag + "act"]), C, n, 0)
    torch.autograd.backward([yi, ya], [_g(g[tag + "dyi"]), _g(g[tag + "dya"])])
    for got, key in ((yi, "yi"), (ya, "ya"), (x.grad, "dx"), (xa.grad, "dxa")):
        assert O.rel_err(got.detach().cpu()[live], torch.from_numpy(g[tag + key])[live]) < TOL, key
    assert O.rel_err(W.grad.cpu(), torch.from_numpy(g[tag + "dW0"])) < TOL
