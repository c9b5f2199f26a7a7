"""Levels of the radix-n digit grouping without index tensors (ncn_forward_radix / ncn_backward_radix) against the
oracle run on the tables of oracle.radix_group_table, and against the library's own table path."""
import ctypes

import pytest
import torch

from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import ncn_cuda_module
    return ncn_cuda_module


def _plan(shape5, first, count, backward):
    from ncn_cuda_amd import _lib
    batch, N, E, C, n = shape5
    sh = _lib.NcnShape(batch, N, E, C, n)
    buf = (ctypes.c_int32 * (6 * 16))()
    k = _lib.load().ncn_plan_radix(ctypes.byref(sh), first, count, 0, int(backward), buf, 16)
    assert k >= 0, k
    return [tuple(buf[6 * i:6 * i + 6]) for i in range(k)]


# (batch, N, E, heads, n_cache, first_level, levels)
CASES = [
    (2, 64, 64, 2, 2, 0, 6),       # every level of N = 2^6: one LDS pass forward, one backward
    (3, 1024, 128, 4, 2, 0, 10),   # 10 levels: two passes each way
    (2, 1024, 64, 2, 2, 3, 5),     # a range that starts at level 3
    (2, 256, 64, 4, 4, 0, 4),      # n = 4, head width 16
    (2, 4096, 128, 4, 4, 1, 5),    # n = 4: levels 1..5 of 4^6
    (2, 96, 32, 2, 2, 0, 5),       # N = 3 * 2^5: windows that do not fill the LDS budget evenly
    (1, 640, 128, 4, 2, 0, 2),     # 160 windows of 4 rows forward, 64 fit a workgroup: 40 per load, 4 loads
    (1, 384, 128, 4, 2, 0, 7),     # N = 3 * 2^7: three windows of 128 rows, the backward budget takes one per load
    (2, 768, 64, 2, 4, 0, 3),      # n = 4, N = 12 * 4^3: 12 windows, 4 per load forward, 2 per load backward
    (2, 512, 32, 2, 8, 0, 3),      # n = 8: no LDS passes, closed-form positions in the one-stage register kernels
    (2, 81, 10, 2, 3, 0, 4),       # n = 3, head width 5: generic kernel
    (2, 128, 256, 2, 2, 2, 3),     # head width 128: register kernels, one level per launch
    (2, 64, 16, 16, 2, 0, 6),      # one feature per head, laid out as one head of 16: levels in LDS like heads of 16
    (2, 1024, 64, 64, 4, 0, 5),    # the same at n = 4, two "heads" of 32
    (2, 512, 8, 8, 8, 0, 3),       # one feature per head at n = 8: one level per launch
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_N%d_E%d_C%d_n%d_l%d_L%d" % c)
def test_radix_levels_vs_oracle_tables(M, case):
    batch, N, E, C, n, first, L = case
    alpha = 0.9
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=41, xa_zero=False)
    tables = [O.radix_group_table(N, n, first + l) for l in range(L)]
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), alpha, n, C, tables)
    gx, gxa, gdy, gdya = x.cuda(), xa.cuda(), dy.cuda(), dya.cuda()
    W = torch.stack(Ws).cuda()
    y, ya = M.forward_radix(gx, gxa, W, alpha, 0, n, C, first, L)
    assert O.rel_err(y, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5
    xr, xar, dx, dxa, dW = M.backward_radix(y, ya, gdy, gdya, W, alpha, 0, n, C, first, L)
    tol = max(1e-5, 2e-6 * (1 / 0.9) ** (n * L))        # whole-range reversal
    assert O.rel_err(dx, ref[2]) < tol and O.rel_err(dxa, ref[3]) < tol
    for l in range(L):
        assert O.rel_err(dW[l], ref[4][l]) < tol, f"dW{l}"
    assert O.rel_err(xr, x) < tol and O.rel_err(xar, xa) < tol
    # without the reconstructed inputs (state through the workspace, the last pass writes gradients only): same bits
    lean = M.backward_radix(y, ya, gdy, gdya, W, alpha, 0, n, C, first, L, want_inputs=False)
    assert lean[0] is None and torch.equal(lean[2], dx) and torch.equal(lean[3], dxa) and torch.equal(lean[4], dW)
    ix, ixa = M.inverse_radix(y, ya, W, alpha, 0, n, C, first, L)
    assert O.rel_err(ix, x) < tol and O.rel_err(ixa, xa) < tol
    # the table path of the library on the same levels (one launch per level): rounding-level agreement
    gt = torch.stack(tables).to(torch.int32).cuda()
    ty, tya = M.forward_stages(gx, gxa, W, alpha, 0, n, C, 0, L, group_index=gt)
    assert O.rel_err(y, ty) < 2e-6 and O.rel_err(ya, tya) < 2e-6


def test_radix_plans_and_errors(M):
    # N = 8192, n = 2, 13 levels: 8 + 5 forward (256-row windows), 7 + 6 backward (128-row windows)
    fwd = _plan((128, 8192, 128, 4, 2), 0, 13, False)
    bwd = _plan((128, 8192, 128, 4, 2), 0, 13, True)
    assert [(p[0], p[1], p[2]) for p in fwd] == [(0, 8, 1), (8, 5, 1)]
    assert [(p[0], p[1], p[2]) for p in bwd] == [(0, 7, 1), (7, 6, 1)]
    assert fwd[0][3:] == (1, 256, 256) and fwd[1][3:] == (256, 32, 256)
    # n = 8 has no LDS build: one launch per level
    assert [(p[1], p[2]) for p in _plan((2, 512, 32, 2, 8), 0, 3, False)] == [(1, 0)] * 3
    x = torch.zeros(2, 96, 32, device="cuda")
    with pytest.raises(ValueError, match="divide"):
        M.forward_radix(x, x, torch.zeros(6, 64, device="cuda"), 0.9, 0, 2, 2, 0, 6)      # 2^6 does not divide 96


def test_radix_bf16_input_and_other_activation(M):
    batch, N, E, C, n, L = 2, 512, 64, 2, 2, 9
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=42, xa_zero=False, dtype=torch.bfloat16)
    tables = [O.radix_group_table(N, n, l) for l in range(L)]
    f = torch.float32
    ref = O.net_autograd_indexed(x.to(f).double(), xa.to(f).double(), [w.to(f).double() for w in Ws], dy.to(f).double(),
                                 dya.to(f).double(), 0.9, n, C, tables, activation=2)
    W = torch.stack(Ws).cuda()
    y, ya = M.forward_radix(x.cuda(), xa.cuda(), W, 0.9, 2, n, C, 0, L)
    assert y.dtype == torch.float32
    assert O.rel_err(y, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5   # bf16 inputs are exact in float32
    _, _, dx, dxa, dW = M.backward_radix(y, ya, dy.cuda(), dya.cuda(), W, 0.9, 2, n, C, 0, L)
    tol = 2e-6 * (1 / 0.9) ** (n * L)
    assert O.rel_err(dx, ref[2]) < tol and O.rel_err(dW[0], ref[4][0]) < tol and O.rel_err(dW[L - 1], ref[4][L - 1]) < tol


def test_radix_net_autograd_node(M):
    """fused_ncn_radix_net through torch autograd, bf16 in and out, segments of 26 // n levels."""
    import ncn_cuda_amd as pkg
    batch, N, E, C, n, L = 2, 4096, 64, 2, 4, 6          # 4^6 = 4096; two saved segments of three levels
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=43, xa_zero=False)
    tables = [O.radix_group_table(N, n, l) for l in range(L)]
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, tables)
    gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
    gw = [w.cuda().requires_grad_() for w in Ws]
    yi, ya = pkg.fused_ncn_radix_net(gx, gxa, gw, 0.9, 0, n, C, save_every=3)
    torch.autograd.backward([yi, ya], [dy.cuda(), dya.cuda()])
    tol = 2e-6 * (1 / 0.9) ** (n * 3)
    assert O.rel_err(yi, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5
    assert O.rel_err(gx.grad, ref[2]) < tol and O.rel_err(gxa.grad, ref[3]) < tol
    for l in range(L):
        assert gw[l].grad.shape == gw[l].shape and O.rel_err(gw[l].grad, ref[4][l]) < tol


def test_net_modules_with_radix_grouping(M):
    import ncn_cuda_amd as pkg
    batch, N, E, C, n, L = 2, 256, 64, 2, 2, 8
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=44, xa_zero=False)
    tables = [O.radix_group_table(N, n, l) for l in range(L)]
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, tables)
    gw = [w.cuda().requires_grad_() for w in Ws]
    net = pkg.NCNNetTestCuda(0.9, "tanh", n, C, L, gw, grouping="radix")
    gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
    yi, ya = net(gx, gxa)
    torch.autograd.backward([yi, ya], [dy.cuda(), dya.cuda()])
    assert O.rel_err(yi, ref[0]) < 1e-5 and O.rel_err(gx.grad, ref[2]) < 3e-5 and O.rel_err(gw[3].grad, ref[4][3]) < 3e-5
    mod = pkg.NCNNetCuda(0.9, "tanh", n, C, L, E, grouping="radix").cuda()
    assert sorted(mod.state_dict()) == [f"ncn_modules.{l}.weight" for l in range(L)]
    y2, _ = mod(x.cuda(), xa.cuda())
    assert y2.shape == x.shape and torch.isfinite(y2).all()
    with pytest.raises(ValueError):
        pkg.NCNNetCuda(0.9, "tanh", n, C, L, E, grouping="butterfly")
