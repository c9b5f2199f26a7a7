"""Multi-stage calls (n_stages > 1): the LDS-resident passes must reproduce the one-launch-per-stage path and the
oracle, for closed passes, halo passes, wrapped strides, stage ranges that do not start at 0, and dya = NULL."""
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


# (batch, N, E, C, n, first_stage, L)
CASES = [
    (3, 1024, 64, 2, 2, 0, 11),    # groups 512: halo passes, a closed pass, and strides that wrap to 0 at the end
    (2, 8192, 128, 4, 2, 0, 13),   # the deep small-group configuration at its real N (batch cut down)
    (2, 1024, 128, 4, 4, 0, 5),    # n = 4, 5 stages (groups 256)
    (2, 512, 32, 2, 8, 0, 4),      # n = 8: no LDS passes, the call loops over one-stage launches
    (2, 512, 32, 2, 4, 1, 5),      # n = 4, head width 16
    (2, 2048, 64, 2, 2, 3, 6),     # range that starts at stage 3 (stride 4)
    (1, 256, 32, 1, 2, 0, 8),      # one head; whole ring fits the window from the start
    (5, 64, 128, 4, 4, 0, 3),      # tiny ring (16 groups)
    (2, 256, 64, 2, 2, 1000003, 3),  # a very high first stage: 2^(stage-1) mod groups is 0 from stage log2(groups)+1 on
    (3, 2048, 64, 4, 2, 0, 10),    # n = 2, head width 16 (16 groups per wave tile, windows of 512 groups)
    (2, 16, 32, 1, 2, 0, 3),       # n = 2, 8 groups: a window smaller than one wave tile per wave
    (3, 2048, 16, 2, 2, 0, 10),    # n = 2, head width 8 (one lane per group, 64 groups per wave tile)
    (2, 2048, 128, 2, 2, 0, 11),   # n = 2, head width 64 (windows of 64 groups, backward passes of 3 stages)
    (2, 1024, 32, 4, 4, 0, 6),     # n = 4, head width 8
    (2, 512, 128, 2, 4, 0, 6),     # n = 4, head width 64 (windows of 16 groups)
    (2, 3 * 512, 64, 2, 2, 0, 12),   # 768 groups = 3 * 2^8: strides wrap to 256 and 512 in turn, closed passes on rings of 3, 6, ..
    (2, 96, 32, 4, 4, 0, 6),         # n = 4, 24 groups = 3 * 8
    (1, 3 * 4096, 128, 4, 2, 0, 13), # 6144 groups: halo passes on a ring that is no power of two, then closed ones
    (2, 5 * 256, 64, 2, 2, 0, 9),    # 640 groups = 5 * 2^7
    (2, 7 * 64, 32, 2, 4, 2, 5),     # n = 4, 112 groups = 7 * 16, from stage 2
    (2, 2048, 256, 2, 2, 0, 11),     # n = 2, head width 128 (16 lanes per row, windows of 32 groups)
    (2, 1024, 128, 1, 4, 5, 4),      # n = 4, head width 128: closed passes on the rings of the high stages    # heads of one feature (E == n_head), laid out as heads of 32, 16 and 8 adjacent ones: the same passes
    (2, 8192, 128, 128, 2, 0, 13),   # the deep configuration's N on 128 one-feature heads (4 "heads" of 32)
    (3, 1024, 48, 48, 2, 0, 11),     # E = 3 * 16
    (2, 1024, 128, 128, 4, 0, 5),    # n = 4
    (2, 512, 24, 24, 4, 1, 5),       # n = 4, E = 3 * 8
    (2, 512, 12, 12, 2, 0, 6),       # E = 3 * 4: no LDS passes at four heads to a row, one launch per stage
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d" % c)
def test_multi_stage_matches_single_stage_and_oracle(M, case):
    batch, N, E, C, n, first, L = case
    alpha = 0.9
    x, xa, Ws, dyi, dya = O.make_inputs(batch, N, E, L, n, seed=17, xa_zero=False)
    gx, gxa, gdy, gdya = x.cuda(), xa.cuda(), dyi.cuda(), dya.cuda()
    gWs = [w.cuda() for w in Ws]
    Wst = torch.stack(gWs)
    # one launch per stage
    outs = []
    cx, cxa = gx, gxa
    for l in range(L):
        cx, cxa = M.forward(cx, cxa, gWs[l], alpha, 0, n, C, first + l)
        outs.append((cx, cxa))
    # groups of 2 and 4 rows at heads of 8 to 128 features, an even number of groups: the call really uses LDS passes
    wide = next(w for w in (32, 16, 8, 4, 1) if E % w == 0) if C == E else E // C   # one-feature heads: adjacent heads per row
    if n in (2, 4) and wide in (8, 16, 32, 64, 128) and (N // n) % 2 == 0:
        import ctypes
        from ncn_cuda_amd import _lib
        shape = _lib.NcnShape(batch, N, E, C, n)
        for backward in (0, 1):
            assert _lib.load().ncn_plan_passes(ctypes.byref(shape), first, L, 0, backward, None, 0) >= 1
    # one call for all stages
    y, ya = M.forward_stages(gx, gxa, Wst, alpha, 0, n, C, first, L)
    # same arithmetic up to where the powers of m are folded in (per stage vs per pass): rounding-level agreement
    assert O.rel_err(y, outs[-1][0]) < 2e-6 and O.rel_err(ya, outs[-1][1]) < 2e-6

    d = torch.float64
    ref = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dyi.to(d), dya.to(d), alpha, n, C, first_stage=first)
    assert O.rel_err(y, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5

    xr, xar, dx, dxa, dW = M.backward_stages(y, ya, gdy, gdya, Wst, alpha, 0, n, C, first, L)
    # whole-range reversal: float32 rounding grows like (1/m)^(n L)
    amp = (1 / 0.9) ** (n * L)
    tol = max(1e-5, 5e-7 * amp)
    assert O.rel_err(dx, ref[2]) < tol
    assert O.rel_err(dxa, ref[3]) < tol
    for l in range(L):
        assert O.rel_err(dW[l], ref[4][l]) < tol, f"dW{l}"
    assert O.rel_err(xr, x) < tol
    assert O.rel_err(xar, xa) < tol

    # the same reversal done stage by stage through single-stage calls agrees to rounding
    cy, cya, cg, cga = y, ya, gdy, gdya
    for l in range(L - 1, -1, -1):
        cy, cya, cg, cga, dWl = M.backward_stages(cy, cya, cg, cga, gWs[l], alpha, 0, n, C, first + l, 1)
        assert O.rel_err(dW[l], dWl[0]) < 1e-5
    assert O.rel_err(dx, cg) < tol and O.rel_err(dxa, cga) < tol


def test_multi_stage_dya_none_and_bf16_input(M):
    batch, N, E, C, n, L = 2, 1024, 128, 4, 2, 10
    x, xa, Ws, dyi, _ = O.make_inputs(batch, N, E, L, n, seed=23, xa_zero=True, dtype=torch.bfloat16)
    gx, gxa, gdy = x.cuda(), xa.cuda(), dyi.cuda()
    Wst = torch.stack([w.cuda() for w in Ws])
    y, ya = M.forward_stages(gx, gxa, Wst, 0.9, 0, n, C, 0, L, out_dtype=torch.float32)
    f = torch.float32
    ref = O.net_autograd(x.to(f), xa.to(f), [w.to(f) for w in Ws], dyi.to(f), torch.zeros_like(dyi, dtype=f), 0.9, n, C)
    assert O.rel_err(y, ref[0]) < 2e-5 and O.rel_err(ya, ref[1]) < 2e-5
    a = M.backward_stages(y, ya, gdy, None, Wst, 0.9, 0, n, C, 0, L, grad_dtype=torch.float32)
    b = M.backward_stages(y, ya, gdy, torch.zeros_like(gdy), Wst, 0.9, 0, n, C, 0, L, grad_dtype=torch.float32)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    assert O.rel_err(a[2], ref[2]) < 1e-4
    for l in range(L):
        assert O.rel_err(a[4][l], ref[4][l]) < 1e-4


@pytest.mark.parametrize("act", [1, 2, -1, 3], ids=["relu", "sigmoid", "linear", "leaky_relu"])
@pytest.mark.parametrize("case", [(2, 1024, 64, 2, 2, 0, 9), (2, 512, 128, 4, 4, 1, 4), (2, 512, 64, 64, 4, 0, 4)],
                         ids=["n2_halo_and_closed", "n4_from_stage1", "n4_one_feature_heads"])
def test_multi_stage_other_activations(M, case, act):
    """The LDS passes in their runtime-activation build.  relu and leaky relu have a kink at T = 0, where a float32
    recomputation may pick the other slope: they run on inputs whose T keeps one sign per batch entry (both slopes,
    never near the kink), so every gradient entry is compared."""
    batch, N, E, C, n, first, L = case
    alpha = 0.9
    if act in (1, 3):
        x, xa, Ws, dyi, dya = O.make_inputs_signed_regimes(batch, N, E, L, n, seed=23)
    else:
        x, xa, Ws, dyi, dya = O.make_inputs(batch, N, E, L, n, seed=23, xa_zero=False)
    gx, gxa, gdy, gdya = x.cuda(), xa.cuda(), dyi.cuda(), dya.cuda()
    Wst = torch.stack(Ws).cuda()
    import ctypes
    from ncn_cuda_amd import _lib
    shape = _lib.NcnShape(batch, N, E, C, n)
    assert _lib.load().ncn_plan_passes(ctypes.byref(shape), first, L, act, 0, None, 0) >= 1   # LDS passes are used
    y, ya = M.forward_stages(gx, gxa, Wst, alpha, act, n, C, first, L)
    d = torch.float64
    ref = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dyi.to(d), dya.to(d), alpha, n, C, activation=act,
                         first_stage=first)
    assert O.rel_err(y, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5
    xr, xar, dx, dxa, dW = M.backward_stages(y, ya, gdy, gdya, Wst, alpha, act, n, C, first, L)
    tol = max(1e-5, 5e-7 * (1 / 0.9) ** (n * L))
    # (the sign-regime inputs of relu / leaky relu have xa in [0, 0.5] beside x in [0.5, 1.5]: the error of xa is
    # measured against the smaller of the two scales)
    assert O.rel_err(xr, x) < tol and O.rel_err(xar, xa) < (3 * tol if act in (1, 3) else tol)
    assert O.rel_err(dx, ref[2]) < tol and O.rel_err(dxa, ref[3]) < tol
    for l in range(L):
        assert O.rel_err(dW[l], ref[4][l]) < tol


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d" % c)
def test_multi_stage_inverse(M, case):
    """ncn_inverse over a stage range (LDS passes where they can run without scratch) against one inverse call per
    stage and against the inputs of the forward."""
    batch, N, E, C, n, first, L = case
    alpha = 0.9
    x, xa, Ws, _, _ = O.make_inputs(batch, N, E, L, n, seed=19, xa_zero=False)
    gx, gxa = x.cuda(), xa.cuda()
    Wst = torch.stack(Ws).cuda()
    y, ya = M.forward_stages(gx, gxa, Wst, alpha, 0, n, C, first, L)
    xi, xai = M.inverse_stages(y, ya, Wst, alpha, 0, n, C, first, L)
    tol = max(1e-5, 5e-7 * (1 / 0.9) ** (n * L))
    assert O.rel_err(xi, x) < tol and O.rel_err(xai, xa) < tol
    cy, cya = y, ya
    for l in range(L - 1, -1, -1):
        cy, cya = M.inverse_stages(cy, cya, Wst[l], alpha, 0, n, C, first + l, 1)
    assert O.rel_err(xi, cy) < tol and O.rel_err(xai, cya) < tol
    # in place (x, xa are y, ya): halo passes fall back to one launch per stage
    py, pya = y.clone(), ya.clone()
    from ncn_cuda_amd import _lib
    import ctypes
    shape = _lib.NcnShape(batch, N, E, C, n)
    rc = _lib.load().ncn_inverse(ctypes.c_void_p(py.data_ptr()), ctypes.c_void_p(pya.data_ptr()), 0,
                                 ctypes.c_void_p(py.data_ptr()), ctypes.c_void_p(pya.data_ptr()), 0,
                                 ctypes.c_void_p(Wst.data_ptr()), ctypes.byref(shape), first, L, alpha, 0.9, 0,
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert O.rel_err(py, xi) < tol and O.rel_err(pya, xai) < tol
    # without scratch (ncn_inverse) and with it (ncn_inverse_ws, what inverse_stages calls): same stages, other launches
    xn, xan = M.inverse_stages(y, ya, Wst, alpha, 0, n, C, first, L, scratch=False)
    assert O.rel_err(xn, xi) < tol and O.rel_err(xan, xai) < tol
    # ncn_inverse_ws in place, with the forward's scratch size
    ws_bytes = _lib.load().ncn_workspace_bytes_stages(ctypes.byref(shape), first, L, 0, 0)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")
    qy, qya = y.clone(), ya.clone()
    rc = _lib.load().ncn_inverse_ws(ctypes.c_void_p(qy.data_ptr()), ctypes.c_void_p(qya.data_ptr()), 0,
                                    ctypes.c_void_p(qy.data_ptr()), ctypes.c_void_p(qya.data_ptr()), 0,
                                    ctypes.c_void_p(Wst.data_ptr()), ctypes.c_void_p(ws.data_ptr()),
                                    ctypes.c_size_t(ws_bytes), ctypes.byref(shape), first, L, alpha, 0.9, 0,
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert O.rel_err(qy, xi) < tol and O.rel_err(qya, xai) < tol


def _stage_by_stage_dW(M, outs, gdy, gdya, gWs, alpha, act, n, C, first):
    dWs = [None] * len(gWs)
    dy, dya = gdy, gdya
    for l in range(len(gWs) - 1, -1, -1):
        _, _, dy, dya, dW = M.backward(outs[l][0], outs[l][1], dy, dya, gWs[l], alpha, act, n, C, first + l)
        dWs[l] = dW.reshape(-1)
    return torch.stack(dWs), dy, dya


@pytest.mark.parametrize("case", [
    (2, 256, 8, 2, 2, 0, 11),       # more stages in one call than one reduction job holds (8): two jobs
                                    # (heads of 4 features: no LDS passes, one launch per stage)
    (8192, 64, 128, 4, 16, 0, 2),   # 16384 partial rows per stage: the buffer holds one stage, a job per stage
    (640, 256, 128, 4, 8, 1, 3),    # 5120 rows per stage: three stages side by side (15360 rows), one job
], ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d" % c)
def test_dw_of_a_call_equals_dw_of_its_stages(M, case):
    """The launches of a call write their dW partial rows side by side and are summed together; when the partial
    buffer or the job is full the sums so far are taken first.  Either way each stage's partial rows are added in
    the order a one-stage call adds them: bit-identical dW."""
    batch, N, E, C, n, first, L = case
    alpha = 0.9
    gen = torch.Generator(device="cuda").manual_seed(3)
    gx = torch.randn(batch, N, E, device="cuda", generator=gen)
    gxa = torch.randn(batch, N, E, device="cuda", generator=gen)
    gdy = torch.randn(batch, N, E, device="cuda", generator=gen)
    gWs = [torch.randn(2 * E, device="cuda", generator=gen) * 0.2 for _ in range(L)]
    outs, cx, cxa = [], gx, gxa
    for l in range(L):
        cx, cxa = M.forward(cx, cxa, gWs[l], alpha, 0, n, C, first + l)
        outs.append((cx, cxa))
    ref_dW, ref_dx, ref_dxa = _stage_by_stage_dW(M, outs, gdy, None, gWs, alpha, 0, n, C, first)
    _, _, dx, dxa, dW = M.backward_stages(outs[-1][0], outs[-1][1], gdy, None, torch.stack(gWs), alpha, 0, n, C, first, L)
    # the call inverts from the last outputs, the stage-by-stage path from each stage's saved outputs: dx agrees to
    # rounding; both run the same one-stage kernels, and dW's sums must not depend on the batching
    assert O.rel_err(dx, ref_dx) < 1e-4 and O.rel_err(dxa, ref_dxa) < 1e-4
    assert O.rel_err(dW, ref_dW) < 1e-4
    # same inputs per stage (top stage reads the same outputs and gradients): its dW is bit-identical
    assert torch.equal(dW[L - 1], ref_dW[L - 1])
    # and a second identical call reproduces every bit
    _, _, _, _, dW2 = M.backward_stages(outs[-1][0], outs[-1][1], gdy, None, torch.stack(gWs), alpha, 0, n, C, first, L)
    assert torch.equal(dW, dW2)


def test_backward_with_the_smaller_workspace_loops_over_windows(M):
    """ncn_backward gives every window of a multi-stage pass a workgroup of its own when the workspace has a dW partial
    row for each (ncn_workspace_bytes_stages); with ncn_workspace_bytes plus the four float32 arrays, which every
    version of the library accepted, the workgroups of a pass that does not fit walk over several windows (the other
    build of the kernel).  Same windows, same arithmetic: dx, dxa and the reconstructed inputs must be bit-identical,
    dW equal up to the order of its partial sums."""
    import ctypes
    from ncn_cuda_amd import _lib
    batch, N, E, C, n, L = 80, 8192, 128, 4, 2, 13     # 80 x 32 closed windows per head x 7 stages > 16384 partial rows
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(batch, N, E, device=dev, generator=g)
    xa = torch.randn(batch, N, E, device=dev, generator=g) * 0.1
    dy = torch.randn(batch, N, E, device=dev, generator=g)
    dya = torch.randn(batch, N, E, device=dev, generator=g)
    W = torch.randn(L, 2 * E, device=dev, generator=g) * (E // C) ** -0.5
    y, ya = M.forward_stages(x, xa, W, 0.9, 0, n, C, 0, L)
    ref = M.backward_stages(y, ya, dy, dya, W, 0.9, 0, n, C, 0, L)

    lib = _lib.load()
    shape = _lib.NcnShape(batch, N, E, C, n)
    plane = (batch * N * E * 4 + 255) // 256 * 256
    small = lib.ncn_workspace_bytes(ctypes.byref(shape)) + 4 * plane
    assert small < lib.ncn_workspace_bytes_stages(ctypes.byref(shape), 0, L, 0, 1)
    ws = torch.empty(small, dtype=torch.uint8, device=dev)
    out = [torch.empty_like(x) for _ in range(4)]       # dx, dxa, x_rec, xa_rec
    dW = torch.empty(L, 2 * E, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.ncn_backward(p(y), p(ya), 0, p(dy), p(dya), 0, p(out[0]), p(out[1]), 0, p(out[2]), p(out[3]), p(W), p(dW),
                          p(ws), ctypes.c_size_t(small), ctypes.byref(shape), 0, L, 0.9, 0.9, 0,
                          ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out[2], ref[0]) and torch.equal(out[3], ref[1])
    assert torch.equal(out[0], ref[2]) and torch.equal(out[1], ref[3])
    assert O.rel_err(dW, ref[4]) < 1e-6
    assert O.rel_err(ref[0], x) < 1e-4      # and both are the inputs again (26 steps undone)

    # the same with one context length per batch entry (the LENGTHS builds of both forms of the kernel)
    lens = torch.tensor([(37 * b * b + 11) % (N + 1) for b in range(batch)], dtype=torch.int32, device=dev)
    y, ya = M.forward_stages(x, xa, W, 0.9, 0, n, C, 0, L, ctx_len=lens)
    ref = M.backward_stages(y, ya, dy, dya, W, 0.9, 0, n, C, 0, L, ctx_len=lens)
    rc = lib.ncn_backward_indexed(p(y), p(ya), 0, p(dy), p(dya), 0, p(out[0]), p(out[1]), 0, p(out[2]), p(out[3]), p(W),
                                  p(dW), p(ws), ctypes.c_size_t(small), None, p(lens), ctypes.byref(shape), 0, L, 0.9,
                                  0.9, 0, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out[2], ref[0]) and torch.equal(out[3], ref[1])
    assert torch.equal(out[0], ref[2]) and torch.equal(out[1], ref[3])
    assert O.rel_err(dW, ref[4]) < 1e-6


@pytest.mark.parametrize("case", [
    (3, 1024, 64, 2, 2, 0, 11),    # several multi-stage passes (halo and closed)
    (1, 256, 32, 1, 2, 0, 8),      # one pass covers the range
    (2, 1024, 128, 4, 4, 0, 5),    # multi-stage passes and one-stage launches mixed
    (2, 512, 32, 2, 8, 0, 4),      # one-stage launches only
    (2, 96, 20, 2, 3, 1, 3),       # the generic kernels
    (3, 1024, 32, 32, 2, 0, 11),   # heads of one feature: several multi-stage passes
], ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d" % c)
@pytest.mark.parametrize("grouping", ["closed", "lengths", "table"])
def test_backward_without_reconstructed_inputs(M, case, grouping):
    """x_rec = xa_rec = NULL with several stages: the state between the stages travels through the workspace and the
    last stage to run writes no reconstructed inputs.  Same kernels on the same values: dx, dxa, dW bit-identical to
    the call that returns them."""
    batch, N, E, C, n, first, L = case
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=29, xa_zero=False)
    gx, gxa, gdy, gdya = x.cuda(), xa.cuda(), dy.cuda(), dya.cuda()
    W = torch.stack(Ws).cuda()
    kw = {}
    if grouping == "lengths":
        kw["ctx_len"] = torch.tensor(([N // 2 + 1, N, 3, 0, N - 1])[:batch], dtype=torch.int32).cuda()
    if grouping == "table":
        kw["group_index"] = torch.stack([O.stride_group_table(N, n, first + l) for l in range(L)]).to(torch.int32).cuda()
        first = 0
    y, ya = M.forward_stages(gx, gxa, W, 0.9, 0, n, C, first, L, **kw)
    full = M.backward_stages(y, ya, gdy, gdya, W, 0.9, 0, n, C, first, L, **kw)
    lean = M.backward_stages(y, ya, gdy, gdya, W, 0.9, 0, n, C, first, L, want_inputs=False, **kw)
    assert lean[0] is None and lean[1] is None
    for k in (2, 3, 4):
        assert torch.equal(full[k], lean[k])
    # and without the workspace for it the call says so instead of running
    import ctypes
    from ncn_cuda_amd import _lib
    lib = _lib.load()
    shape = _lib.NcnShape(batch, N, E, C, n)
    small = lib.ncn_workspace_bytes(ctypes.byref(shape))
    ws = torch.empty(small, dtype=torch.uint8, device="cuda")
    dx, dxa, dW = torch.empty_like(gx), torch.empty_like(gx), torch.empty(L, 2 * E, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    if grouping == "closed" and lib.ncn_plan_passes(ctypes.byref(shape), first, L, 0, 1, None, 0) != 1:
        rc = lib.ncn_backward(p(y), p(ya), 0, p(gdy), p(gdya), 0, p(dx), p(dxa), 0, None, None, p(W), p(dW), p(ws),
                              ctypes.c_size_t(small), ctypes.byref(shape), first, L, 0.9, 0.9, 0,
                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == -8
