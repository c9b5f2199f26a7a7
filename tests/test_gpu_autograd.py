"""The reference's autograd / nn.Module surface on the GPU: same names, same call pattern as
grad_test_bench.py:116-134, results against the CPU oracle."""
import pytest
import torch

from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import ncn_cuda_amd
    return ncn_cuda_amd


def test_net_test_cuda_like_reference_script(pkg):
    # the reference script's own configuration, grad_test_bench.py:22-32
    batch, n_head, N, E, alpha, n, L = 4, 4, 256, 128, 0.9, 32, 3
    g = torch.Generator().manual_seed(0)
    x = (0.5 * torch.randn(batch, N, E, generator=g))
    xa = torch.zeros(batch, N, E)
    Ws = [0.5 * torch.randn(2 * E, generator=g) for _ in range(L)]
    dyi = torch.randn(batch, N, E, generator=g)
    d = torch.float64
    ref_yi, ref_ya, ref_dx, ref_dxa, ref_dWs = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dyi.to(d),
                                                              torch.zeros_like(dyi, dtype=d), alpha, n, n_head)
    gx = x.cuda().requires_grad_()
    gxa = xa.cuda().requires_grad_()
    gWs = [w.cuda().requires_grad_() for w in Ws]
    net = pkg.NCNNetTestCuda(alpha, "tanh", n, n_head, L, gWs)
    yi, ya = net(gx, gxa)
    yi.backward(dyi.cuda())
    assert O.rel_err(yi, ref_yi) < 1e-5
    assert O.rel_err(ya, ref_ya) < 1e-5
    # n_cache = 32 amplifies inversion rounding by (1/0.9)^32 = 29: the reference's own check uses atol=1e-2
    # (grad_test_bench.py:161); float32 still lands near 1e-5 relative (measured: dx 4.1e-6, worst dW 1.5e-5)
    from conftest import record_errors
    record_errors("reference_script_shape", n=n, amp=(1 / 0.9) ** n, dx=O.rel_err(gx.grad, ref_dx),
                  dxa=O.rel_err(gxa.grad, ref_dxa), dW=max(O.rel_err(gWs[l].grad, ref_dWs[l]) for l in range(L)))
    assert O.rel_err(gx.grad, ref_dx) < 3e-5
    assert O.rel_err(gxa.grad, ref_dxa) < 3e-5
    for l in range(L):
        assert O.rel_err(gWs[l].grad, ref_dWs[l]) < 3e-5


def test_net_cuda_module_list_and_state_dict(pkg):
    alpha, n, C, L, E = 0.9, 4, 4, 3, 32
    torch.manual_seed(0)
    net = pkg.NCNNetCuda(alpha, "tanh", n, C, L, E).cuda()
    assert sorted(net.state_dict().keys()) == [f"ncn_modules.{l}.weight" for l in range(L)]
    with torch.no_grad():
        for mod in net.ncn_modules:
            mod.weight.normal_(0, 0.5)
    x = torch.randn(2, 64, E, device="cuda", requires_grad=True)
    xa = torch.randn(2, 64, E, device="cuda", requires_grad=True)
    yi, ya = net(x, xa)
    (yi.sum() + 2 * ya.sum()).backward()
    d = torch.float64
    Ws = [mod.weight.detach().cpu().to(d) for mod in net.ncn_modules]
    ones = torch.ones(2, 64, E, dtype=d)
    ref_yi, ref_ya, ref_dx, ref_dxa, ref_dWs = O.net_autograd(x.detach().cpu().to(d), xa.detach().cpu().to(d), Ws,
                                                              ones, 2 * ones, alpha, n, C)
    assert O.rel_err(yi, ref_yi) < 1e-5
    assert O.rel_err(x.grad, ref_dx) < 1e-5
    assert O.rel_err(xa.grad, ref_dxa) < 1e-5
    for l in range(L):
        assert O.rel_err(net.ncn_modules[l].weight.grad, ref_dWs[l]) < 1e-5


def test_bf16_autograd(pkg):
    batch, N, E, C, n, L, alpha = 2, 128, 128, 4, 16, 3, 0.9
    x, xa, Ws, dyi, dya = O.make_inputs(batch, N, E, L, n, seed=4, xa_zero=True, dtype=torch.bfloat16)
    f = torch.float32
    ref_yi, ref_ya, ref_dx, ref_dxa, ref_dWs = O.net_autograd(x.to(f), xa.to(f), [w.to(f) for w in Ws], dyi.to(f),
                                                              dya.to(f), alpha, n, C)
    gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
    gWs = [w.cuda().requires_grad_() for w in Ws]
    net = pkg.NCNNetTestCuda(alpha, "tanh", n, C, L, gWs)
    yi, ya = net(gx, gxa)
    assert yi.dtype == torch.bfloat16
    torch.autograd.backward([yi, ya], [dyi.cuda(), dya.cuda()])
    assert O.rel_err(yi, ref_yi) < 2e-2
    assert O.rel_err(gx.grad, ref_dx) < 2e-2
    assert O.rel_err(gxa.grad, ref_dxa) < 2e-2
    for l in range(L):
        assert gWs[l].grad.dtype == torch.bfloat16
        assert O.rel_err(gWs[l].grad, ref_dWs[l]) < 2e-2


@pytest.mark.parametrize("cfg", [(2, 1024, 128, 4, 2, 9, torch.float32), (2, 512, 128, 4, 4, 7, torch.float32),
                                 (2, 256, 128, 4, 16, 3, torch.bfloat16), (2, 512, 64, 2, 2, 6, torch.bfloat16),
                                 (2, 512, 64, 64, 2, 7, torch.float32), (2, 256, 128, 128, 16, 3, torch.bfloat16)],
                         ids=["n2_L9_f32", "n4_L7_f32", "n16_L3_bf16", "n2_L6_bf16", "n2_L7_f32_one_feature_heads",
                              "n16_L3_bf16_one_feature_heads"])
def test_whole_net_node_matches_oracle_and_per_stage_nodes(pkg, cfg):
    """NCNNetFunction (one node for the stack, checkpoints every save_every stages) against the oracle and against
    the reference-style chain of per-stage nodes."""
    batch, N, E, C, n, L, dtype = cfg
    alpha = 0.9
    x, xa, Ws, dyi, dya = O.make_inputs(batch, N, E, L, n, seed=31, xa_zero=False, dtype=dtype)
    f = torch.float64 if dtype == torch.float32 else torch.float32
    ref = O.net_autograd(x.to(f), xa.to(f), [w.to(f) for w in Ws], dyi.to(f), dya.to(f), alpha, n, C)
    tol = 2e-5 if dtype == torch.float32 else 2e-2

    def run(fuse):
        gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
        gWs = [w.cuda().requires_grad_() for w in Ws]
        net = pkg.NCNNetTestCuda(alpha, "tanh", n, C, L, gWs, fuse_stages=fuse)
        yi, ya = net(gx, gxa)
        assert yi.dtype == dtype
        torch.autograd.backward([yi, ya], [dyi.cuda(), dya.cuda()])
        return yi, ya, gx.grad, gxa.grad, [w.grad for w in gWs]

    fused, chain = run(True), run(False)
    for got in (fused, chain):
        assert O.rel_err(got[0], ref[0]) < tol and O.rel_err(got[1], ref[1]) < tol
        assert O.rel_err(got[2], ref[2]) < tol and O.rel_err(got[3], ref[3]) < tol
        for l in range(L):
            assert got[4][l].dtype == dtype
            assert O.rel_err(got[4][l], ref[4][l]) < tol, f"dW{l}"
    assert pkg.default_save_every(2) == 13 and pkg.default_save_every(16) == 1
    # groups of 8 rows and more keep every stage's outputs while they fit the memory budget, segments beyond it
    assert pkg.default_save_every(8) == 3 and pkg.default_save_every(8, 4, 1 << 24) == 1
    assert pkg.default_save_every(8, 4, 1 << 24, budget_bytes=1 << 20) == 3 and pkg.default_save_every(2, 13, 1 << 24) == 13


def test_net_cuda_fuse_stages_flag_keeps_parameters(pkg):
    torch.manual_seed(1)
    a = pkg.NCNNetCuda(0.9, "tanh", 2, 4, 6, 128).cuda()
    b = pkg.NCNNetCuda(0.9, "tanh", 2, 4, 6, 128, fuse_stages=True).cuda()
    with torch.no_grad():
        for m in a.ncn_modules:
            m.weight.normal_(0, 0.5)
    b.load_state_dict(a.state_dict())
    x = torch.randn(2, 256, 128, device="cuda")
    xa = torch.randn(2, 256, 128, device="cuda")
    xs = [x.clone().requires_grad_() for _ in range(2)]
    outs = []
    for net, xi in zip((a, b), xs):
        yi, ya = net(xi, xa)
        (yi.square().sum() + ya.sum()).backward()
        outs.append((yi, xi.grad, [m.weight.grad for m in net.ncn_modules]))
    assert O.rel_err(outs[1][0], outs[0][0]) < 1e-6
    assert O.rel_err(outs[1][1], outs[0][1]) < 1e-5
    for ga, gb in zip(outs[0][2], outs[1][2]):
        assert O.rel_err(gb, ga) < 1e-5


def test_triton_named_surface_matches_cuda_named_surface(pkg):
    """NCNNetTestTriton (activation by name) and NCNNetTestCuda give the same numbers: one set of kernels."""
    from ncn_cuda_amd import ncn_triton as T
    batch, N, E, C, n, L = 2, 128, 64, 2, 8, 3
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=3, xa_zero=False)
    for name in ("tanh", "leaky-relu", "identity"):
        res = []
        for make in (lambda w: T.NCNNetTestTriton(0.9, name, n, C, L, w),
                     lambda w: pkg.NCNNetTestCuda(0.9, name if name in pkg.ACTIVATION_CODES else "linear", n, C, L, w)):
            gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
            gw = [w.cuda().requires_grad_() for w in Ws]
            yi, ya = make(gw)(gx, gxa)
            torch.autograd.backward([yi, ya], [dy.cuda(), dya.cuda()])
            res.append([yi, ya, gx.grad, gxa.grad] + [w.grad for w in gw])
        for a, b in zip(*res):
            assert torch.equal(a, b)
    d = torch.float64
    ref = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, activation=-1)
    assert O.rel_err(res[0][0], ref[0]) < 1e-5 and O.rel_err(res[0][2], ref[2]) < 1e-5


@pytest.mark.parametrize("fuse", [False, True], ids=["per_stage_nodes", "one_node"])
def test_missing_upstream_gradients_are_not_materialised(pkg, fuse):
    """yi.backward(dyi) (grad_test_bench.py:121) leaves ya without a gradient: the nodes take None for it (no tensor of
    zeros is made) and give what explicit zeros give, bit for bit; only dya works too, and neither gives no gradient."""
    batch, N, E, C, n, L = 2, 128, 128, 4, 4, 3
    x, xa, Ws, dyi, dya = O.make_inputs(batch, N, E, L, n, seed=5, xa_zero=False)

    def run(which):
        gx, gxa = x.cuda().requires_grad_(), xa.cuda().requires_grad_()
        gWs = [w.cuda().requires_grad_() for w in Ws]
        yi, ya = pkg.NCNNetTestCuda(0.9, "tanh", n, C, L, gWs, fuse_stages=fuse)(gx, gxa)
        if which == "yi":
            yi.backward(dyi.cuda())
        elif which == "ya":
            ya.backward(dya.cuda())
        elif which == "yi_zeros":
            torch.autograd.backward([yi, ya], [dyi.cuda(), torch.zeros_like(ya)])
        else:
            torch.autograd.backward([yi, ya], [torch.zeros_like(yi), dya.cuda()])
        return [gx.grad, gxa.grad] + [w.grad for w in gWs]

    for a, b in zip(run("yi"), run("yi_zeros")):
        assert torch.equal(a, b)
    for a, b in zip(run("ya"), run("zeros_ya")):
        assert torch.equal(a, b)
