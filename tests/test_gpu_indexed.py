"""Table-grouped stages and per-batch context lengths on the GPU (ncn_forward_indexed / ncn_backward_indexed /
ncn_inverse_indexed through the C ABI) against the CPU oracle.  float32, 1e-5 relative unless stated."""
import pytest
import torch

from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-5


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import ncn_cuda_module
    return ncn_cuda_module


def _dev(*ts):
    return [t.cuda() if t is not None else None for t in ts]


def _tables(kind, N, n, L):
    if kind == "stride":
        return [O.stride_group_table(N, n, l) for l in range(L)]
    if kind == "radix":
        levels = 0
        while n ** (levels + 1) <= N and N % (n ** (levels + 1)) == 0:
            levels += 1
        return [O.radix_group_table(N, n, l % levels) for l in range(L)]
    g = torch.Generator().manual_seed(99)
    return [torch.randperm(N, generator=g) for _ in range(L)]


def _run_gpu(M, x, xa, Ws, dy, dya, alpha, n, C, tables, lens, act=0, one_call=False):
    gx, gxa, gdy, gdya = _dev(x, xa, dy, dya)
    gW = torch.stack(Ws).cuda()
    gt = torch.stack(tables).to(torch.int32).cuda()
    gl = torch.tensor(lens, dtype=torch.int32).cuda() if lens is not None else None
    L = len(Ws)
    if one_call:
        y, ya = M.forward_stages(gx, gxa, gW, alpha, act, n, C, 0, L, group_index=gt, ctx_len=gl)
        xr, xar, dx, dxa, dW = M.backward_stages(y, ya, gdy, gdya, gW, alpha, act, n, C, 0, L, group_index=gt,
                                                 ctx_len=gl)
        return y, ya, xr, xar, dx, dxa, [dW[l] for l in range(L)]
    outs = []
    cy, cya = gx, gxa
    for l in range(L):
        cy, cya = M.forward_stages(cy, cya, gW[l], alpha, act, n, C, 0, 1, group_index=gt[l], ctx_len=gl)
        outs.append((cy, cya))
    dWs = [None] * L
    g, h = gdy, gdya
    for l in range(L - 1, -1, -1):
        xr, xar, g, h, dW = M.backward_stages(outs[l][0], outs[l][1], g, h, gW[l], alpha, act, n, C, 0, 1,
                                              group_index=gt[l], ctx_len=gl)
        dWs[l] = dW[0]
    return outs[-1][0], outs[-1][1], xr, xar, g, h, dWs


def _check(got, ref, x, xa, tol=TOL, n=4):
    """Forward at `tol`; what goes through the inversion is allowed its rounding growth (1/m)^n per stage."""
    y, ya, xr, xar, dx, dxa, dWs = got
    ryi, rya, rdx, rdxa, rdWs = ref
    assert O.rel_err(y, ryi) < tol and O.rel_err(ya, rya) < tol
    gtol = max(tol, 1e-6 * (1 / 0.9) ** n)
    assert O.rel_err(dx, rdx) < gtol and O.rel_err(dxa, rdxa) < gtol
    for a, b in zip(dWs, rdWs):
        assert O.rel_err(a, b) < gtol
    if xr is not None:
        rtol = max(3e-5, 3e-6 * (1 / 0.9) ** n)
        assert O.rel_err(xr, x) < rtol and O.rel_err(xar, xa) < rtol


SHAPES = [(3, 64, 32, 2, 4, 3), (2, 256, 128, 4, 16, 2), (3, 36, 20, 2, 3, 3), (5, 128, 64, 2, 8, 2),
          (2, 64, 256, 2, 8, 2), (2, 128, 8, 2, 32, 1), (3, 64, 8, 8, 4, 3), (2, 128, 16, 16, 16, 2)]
IDS = ["register_n4_Ec16", "register_n16_Ec32", "generic_n3_Ec10", "register_n8_Ec32", "register_n8_Ec128",
       "register_n32_Ec4", "register_n4_Ec1", "register_n16_Ec1"]


@pytest.mark.parametrize("kind", ["stride", "radix", "random"])
@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
def test_table_grouping_vs_oracle(M, shape, kind):
    batch, N, E, C, n, L = shape
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=31, xa_zero=False)
    tables = _tables(kind, N, n, L)
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, tables)
    _check(_run_gpu(M, x, xa, Ws, dy, dya, 0.9, n, C, tables, None), ref, x, xa, n=n)


@pytest.mark.parametrize("shape", SHAPES[:2], ids=IDS[:2])
def test_stride_table_equals_closed_form_bit_for_bit(M, shape):
    """The table only replaces the address computation: same kernels, same arithmetic."""
    batch, N, E, C, n, L = shape
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=32, xa_zero=False)
    gx, gxa, gdy, gdya = _dev(x, xa, dy, dya)
    for l in range(L):
        gw = Ws[l].cuda()
        t = O.stride_group_table(N, n, l).to(torch.int32).cuda()
        a = M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, l, 1)
        b = M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, group_index=t)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        ba = M.backward_stages(a[0], a[1], gdy, gdya, gw, 0.9, 0, n, C, l, 1)
        bb = M.backward_stages(a[0], a[1], gdy, gdya, gw, 0.9, 0, n, C, 0, 1, group_index=t)
        for u, v in zip(ba, bb):
            assert torch.equal(u, v)
        ia = M.inverse_stages(a[0], a[1], gw, 0.9, 0, n, C, l, 1)
        ib = M.inverse_stages(a[0], a[1], gw, 0.9, 0, n, C, 0, 1, group_index=t)
        assert torch.equal(ia[0], ib[0]) and torch.equal(ia[1], ib[1])


@pytest.mark.parametrize("kind", ["stride", "radix"])
@pytest.mark.parametrize("one_call", [False, True], ids=["per_stage", "one_call"])
@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
def test_context_lengths_vs_oracle(M, shape, kind, one_call):
    """Lengths that cut a group, end on a group boundary, are zero, full and beyond N."""
    batch, N, E, C, n, L = shape
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=33, xa_zero=False)
    tables = _tables(kind, N, n, L)
    lens = ([N // 2 + 1, 2 * n, N, 0, N + 5] * 2)[:batch]
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), 0.9, n, C, tables,
                                 lens)
    got = _run_gpu(M, x, xa, Ws, dy, dya, 0.9, n, C, tables, lens, one_call=one_call)
    _check(got, ref, x, xa, tol=TOL if not one_call else 3e-5, n=n)


def test_context_lengths_without_table_and_inverse(M):
    """ctx_len with the closed-form stride permutation (group_index = None), and the indexed inverse."""
    batch, N, E, C, n, L = 3, 64, 32, 2, 4, 3
    x, xa, Ws, _, _ = O.make_inputs(batch, N, E, L, n, seed=34, xa_zero=False)
    lens = [N - 3, 9, N]
    tables = [O.stride_group_table(N, n, l) for l in range(L)]
    ry, rya = O.net_forward_indexed(x.double(), xa.double(), [w.double() for w in Ws], 0.9, n, C, tables, lens)
    gx, gxa = _dev(x, xa)
    gW = torch.stack(Ws).cuda()
    gl = torch.tensor(lens, dtype=torch.int32).cuda()
    y, ya = M.forward_stages(gx, gxa, gW, 0.9, 0, n, C, 0, L, ctx_len=gl)
    assert O.rel_err(y, ry) < TOL and O.rel_err(ya, rya) < TOL
    xi, xai = M.inverse_stages(y, ya, gW, 0.9, 0, n, C, 0, L, ctx_len=gl)
    assert O.rel_err(xi, x) < 3e-5 and O.rel_err(xai, xa) < 3e-5
    gt = torch.stack(tables).to(torch.int32).cuda()
    xi2, xai2 = M.inverse_stages(y, ya, gW, 0.9, 0, n, C, 0, L, group_index=gt, ctx_len=gl)
    # lengths alone go through the multi-stage passes, a table through one launch per stage: equal to rounding
    assert O.rel_err(xi, xi2) < TOL and O.rel_err(xai, xai2) < TOL


LENGTH_PASS_CASES = [
    (3, 1024, 64, 2, 2, 0, 11),    # halo passes, a closed pass, strides that wrap to 0
    (2, 8192, 128, 4, 2, 0, 13),   # the deep small-group configuration at its real N
    (4, 1024, 128, 4, 4, 0, 5),    # n = 4
    (3, 2048, 64, 2, 2, 3, 6),     # range that starts at stage 3
    (5, 64, 128, 4, 4, 0, 3),      # tiny ring
    (3, 2048, 64, 4, 2, 1, 9),     # n = 2, head width 16
    (2, 32, 32, 1, 2, 0, 4),       # n = 2, 16 groups: windows smaller than the workgroup's tiles    (3, 1024, 64, 64, 2, 0, 11),   # heads of one feature (two "heads" of 32 adjacent ones), n = 2
    (4, 1024, 16, 16, 4, 0, 5),    # heads of one feature, n = 4
]


@pytest.mark.parametrize("case", LENGTH_PASS_CASES, ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d" % c)
def test_lengths_inside_multi_stage_passes(M, case):
    """Context lengths with the stride permutation over a stage range: the library runs its multi-stage LDS passes
    (rows past a length stay in LDS, the group a length cuts runs its live steps).  Checked against the same call with
    the permutation given as a table, which runs one launch per stage (the path the oracle tests cover), and on the
    smaller cases against the oracle itself."""
    batch, N, E, C, n, first, L = case
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=41, xa_zero=False)
    lens = ([N // 2 + 1, 2 * n, N, 0, N + 5, 1, N - 1] * 2)[:batch]
    tables = [O.stride_group_table(N, n, first + l) for l in range(L)]
    gx, gxa, gdy, gdya = _dev(x, xa, dy, dya)
    gW = torch.stack(Ws).cuda()
    gt = torch.stack(tables).to(torch.int32).cuda()
    gl = torch.tensor(lens, dtype=torch.int32).cuda()
    amp = (1 / 0.9) ** (n * L)
    tol, gtol = 1e-5, max(1e-5, 1e-6 * amp)
    y, ya = M.forward_stages(gx, gxa, gW, 0.9, 0, n, C, first, L, ctx_len=gl)
    ty, tya = M.forward_stages(gx, gxa, gW, 0.9, 0, n, C, 0, L, group_index=gt, ctx_len=gl)
    assert O.rel_err(y, ty) < tol and O.rel_err(ya, tya) < tol
    # rows past the lengths in every stage come out as they went in
    for b, ln in enumerate(lens):
        if ln == 0:
            assert O.rel_err(y[b], gx[b]) < 1e-6 and O.rel_err(ya[b], gxa[b]) < 1e-6
    got = M.backward_stages(y, ya, gdy, gdya, gW, 0.9, 0, n, C, first, L, ctx_len=gl)
    ref = M.backward_stages(y, ya, gdy, gdya, gW, 0.9, 0, n, C, 0, L, group_index=gt, ctx_len=gl)
    for name, u, v in zip(("x_rec", "xa_rec", "dx", "dxa", "dW"), got, ref):
        assert O.rel_err(u, v) < gtol, name
    xi, xai = M.inverse_stages(y, ya, gW, 0.9, 0, n, C, first, L, ctx_len=gl)
    assert O.rel_err(xi, got[0]) < gtol and O.rel_err(xai, got[1]) < gtol
    assert O.rel_err(xi, x) < max(3e-5, 3e-6 * amp)
    if batch * N * E * L <= 3 * 1024 * 64 * 11:
        d = torch.float64
        ry, rya, rdx, rdxa, rdWs = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d),
                                                          dya.to(d), 0.9, n, C, tables, lens)
        assert O.rel_err(y, ry) < tol and O.rel_err(ya, rya) < tol
        assert O.rel_err(got[2], rdx) < gtol and O.rel_err(got[3], rdxa) < gtol
        for l in range(L):
            assert O.rel_err(got[4][l], rdWs[l]) < gtol, "dW%d" % l


def test_bf16_and_other_activation_with_lengths(M):
    batch, N, E, C, n, L = 4, 128, 64, 2, 8, 2
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=35, xa_zero=False, dtype=torch.bfloat16)
    tables = _tables("radix", N, n, L)
    lens = [77, 128, 8, 3]
    f = torch.float32
    ref = O.net_autograd_indexed(x.to(f), xa.to(f), [w.to(f) for w in Ws], dy.to(f), dya.to(f), 0.9, n, C, tables,
                                 lens, activation=3)
    gx, gxa, gdy, gdya = _dev(x, xa, dy, dya)
    gt = torch.stack(tables).to(torch.int32).cuda()
    gl = torch.tensor(lens, dtype=torch.int32).cuda()
    y, ya, y32, ya32 = M.forward_stages(gx, gxa, Ws[0].cuda(), 0.9, 3, n, C, 0, 1, group_index=gt[0], ctx_len=gl,
                                        save_fp32=True)
    y2, ya2, y232, ya232 = M.forward_stages(y32, ya32, Ws[1].cuda(), 0.9, 3, n, C, 0, 1, group_index=gt[1], ctx_len=gl,
                                            out_dtype=torch.bfloat16, save_fp32=True)
    assert y2.dtype == torch.bfloat16
    assert O.rel_err(y2, ref[0]) < 2e-2 and O.rel_err(ya2, ref[1]) < 2e-2
    _, _, g, h, dW1 = M.backward_stages(y232, ya232, gdy, gdya, Ws[1].cuda(), 0.9, 3, n, C, 0, 1, group_index=gt[1],
                                        ctx_len=gl, want_inputs=False)
    _, _, g, h, dW0 = M.backward_stages(y32, ya32, g, h, Ws[0].cuda(), 0.9, 3, n, C, 0, 1, group_index=gt[0],
                                        ctx_len=gl, want_inputs=False)
    assert g.dtype == torch.bfloat16
    assert O.rel_err(g, ref[2]) < 2e-2 and O.rel_err(h, ref[3]) < 2e-2
    assert O.rel_err(dW0[0], ref[4][0]) < 2e-2 and O.rel_err(dW1[0], ref[4][1]) < 2e-2


def test_bad_tables_and_lengths_are_rejected_or_harmless(M):
    batch, N, E, C, n = 2, 32, 16, 2, 4
    x, xa, Ws, _, _ = O.make_inputs(batch, N, E, 1, n, seed=36, xa_zero=False)
    gx, gxa = _dev(x, xa)
    gw = Ws[0].cuda()
    bad = torch.arange(N, dtype=torch.int32).cuda()
    bad[3] = 4
    with pytest.raises(ValueError):
        M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, group_index=bad)
    with pytest.raises(ValueError):
        M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, group_index=bad[:-1], check_tables=False)
    with pytest.raises(ValueError):
        M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, ctx_len=torch.zeros(3, dtype=torch.int32).cuda())
    with pytest.raises(TypeError):
        M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, ctx_len=torch.zeros(2).cuda())
    # out-of-range entries are clamped inside the kernels: wrong numbers, but the call completes
    wild = torch.arange(N, dtype=torch.int32).cuda()
    wild[0], wild[5] = -7, N + 1000
    y, ya = M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, group_index=wild, check_tables=False)
    torch.cuda.synchronize()
    assert torch.isfinite(y).all()
    # negative and oversized lengths are clamped to [0, N]
    gl = torch.tensor([-5, 10 * N], dtype=torch.int32).cuda()
    y, ya = M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1, ctx_len=gl)
    full = M.forward_stages(gx, gxa, gw, 0.9, 0, n, C, 0, 1)
    assert torch.equal(y[0], gx[0]) and torch.equal(y[1], full[0][1])


def test_chunk_linear_surface_autograd(M):
    """fused_chunk_linear_ncn (argument order of ncn_triton_old.py:362-387) through torch autograd."""
    from ncn_cuda_amd import chunk_linear as CL
    batch, N, E, C, n = 3, 64, 32, 2, 4
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, 1, n, seed=37, xa_zero=False)
    lens = [50, 64, 7]
    table = CL.radix_group_table(N, n, 1, device="cuda")
    d = torch.float64
    for act_name, code in (("tanh", 0), ("leaky-relu", 3), ("none", -1)):
        ref = O.net_autograd_indexed(x.to(d), xa.to(d), [Ws[0].to(d)], dy.to(d), dya.to(d), 0.9, n, C,
                                     [table.cpu().long()], lens, activation=code)
        gx = x.cuda().requires_grad_()
        gxa = xa.cuda().requires_grad_()
        gw = Ws[0].cuda().requires_grad_()
        yi, ya = CL.fused_chunk_linear_ncn(gx, gxa, gw, table, torch.tensor(lens).cuda(), 0.9, act_name, C, n, 0)
        torch.autograd.backward([yi, ya], [dy.cuda(), dya.cuda()])
        assert O.rel_err(yi, ref[0]) < TOL and O.rel_err(ya, ref[1]) < TOL
        assert O.rel_err(gx.grad, ref[2]) < TOL and O.rel_err(gxa.grad, ref[3]) < TOL
        assert gw.grad.shape == gw.shape and O.rel_err(gw.grad, ref[4][0]) < TOL


@pytest.mark.parametrize("act", [2, 3, -1], ids=["sigmoid", "leaky_relu", "linear"])
def test_lengths_inside_multi_stage_passes_other_activations(M, act):
    """The builds of the multi-stage kernels that pick the activation at run time, with context lengths: against the
    table path (one launch per stage) on the same lengths.  Leaky relu on inputs that keep T away from its kink."""
    batch, N, E, C, n, first, L = 3, 512, 64, 2, 2, 0, 6
    if act == 3:
        x, xa, Ws, dy, dya = O.make_inputs_signed_regimes(batch, N, E, L, n, seed=47)
    else:
        x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=47, xa_zero=False)
    lens = [N // 2 + 1, N - 1, 3]
    gx, gxa, gdy, gdya = _dev(x, xa, dy, dya)
    gW = torch.stack(Ws).cuda()
    gt = torch.stack([O.stride_group_table(N, n, l) for l in range(L)]).to(torch.int32).cuda()
    gl = torch.tensor(lens, dtype=torch.int32).cuda()
    tol = max(1e-5, 1e-6 * (1 / 0.9) ** (n * L))
    y, ya = M.forward_stages(gx, gxa, gW, 0.9, act, n, C, first, L, ctx_len=gl)
    ty, tya = M.forward_stages(gx, gxa, gW, 0.9, act, n, C, 0, L, group_index=gt, ctx_len=gl)
    assert O.rel_err(y, ty) < 1e-5 and O.rel_err(ya, tya) < 1e-5
    got = M.backward_stages(y, ya, gdy, gdya, gW, 0.9, act, n, C, first, L, ctx_len=gl)
    ref = M.backward_stages(y, ya, gdy, gdya, gW, 0.9, act, n, C, 0, L, group_index=gt, ctx_len=gl)
    for name, u, v in zip(("x_rec", "xa_rec", "dx", "dxa", "dW"), got, ref):
        assert O.rel_err(u, v) < (3 * tol if name == "xa_rec" else tol), name
    xi, xai = M.inverse_stages(y, ya, gW, 0.9, act, n, C, first, L, ctx_len=gl)
    assert O.rel_err(xi, got[0]) < tol and O.rel_err(xai, got[1]) < 3 * tol


@pytest.mark.parametrize("with_lengths", [False, True], ids=["table", "table_and_lengths"])
def test_chunk_linear_bf16_storage_groups_of_16(M, with_lengths):
    """fused_chunk_linear_ncn with bfloat16 tensors at groups of 16 rows: its autograd node has to keep more than the
    bfloat16 outputs (the inversion amplifies their rounding by (1/m)^16 = 5.4).  bfloat16 storage with float32
    arithmetic at 2e-2 against the float64 oracle on the same bfloat16-rounded inputs."""
    from ncn_cuda_amd import chunk_linear as CL
    batch, N, E, C, n = 3, 256, 128, 4, 16
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, 1, n, seed=43, xa_zero=False, dtype=torch.bfloat16)
    lens = [N - 5, 3 * n, N] if with_lengths else None
    table = CL.radix_group_table(N, n, 1, device="cuda")
    d = torch.float64
    ref = O.net_autograd_indexed(x.to(d), xa.to(d), [Ws[0].to(d)], dy.to(d), dya.to(d), 0.9, n, C,
                                 [table.cpu().long()], lens)
    gx = x.cuda().requires_grad_()
    gxa = xa.cuda().requires_grad_()
    gw = Ws[0].cuda().requires_grad_()
    gl = torch.tensor(lens).cuda() if lens is not None else None
    yi, ya = CL.fused_chunk_linear_ncn(gx, gxa, gw, table, gl, 0.9, "tanh", C, n, 0)
    assert yi.dtype == torch.bfloat16
    torch.autograd.backward([yi, ya], [dy.cuda(), dya.cuda()])
    tol = 2e-2
    assert O.rel_err(yi.float(), ref[0]) < tol and O.rel_err(ya.float(), ref[1]) < tol
    assert gx.grad.dtype == torch.bfloat16
    assert O.rel_err(gx.grad.float(), ref[2]) < tol and O.rel_err(gxa.grad.float(), ref[3]) < tol
    assert O.rel_err(gw.grad.float(), ref[4][0]) < tol
