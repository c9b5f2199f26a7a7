"""The four benchmark configurations at their full sizes.  The oracle cannot run them whole, so parity is carried by what
does not depend on size: (batch, head) instances are independent, hence the first batch entries of a full-size run
must equal the oracle on just those entries; dW is a sum over batch entries, hence the full-size dW must equal the
sum of the dW of batch chunks; inverse(forward(x)) must give x back; two runs must agree bit for bit."""
import json
import os

import pytest
import torch

from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu

# name: batch, N, E, heads, n_cache, stages, storage dtype, W scale   (the shapes bench.py runs)
CONFIGS = {
    "cfg2": (32, 1024, 128, 4, 4, 5, torch.float32, 1.0),
    "cfg3": (128, 4096, 128, 4, 16, 3, torch.bfloat16, 1.0),
    "cfg4": (128, 8192, 128, 4, 2, 13, torch.float32, 1.0),
    "cfg5": (64, 2048, 128, 4, 8, 4, torch.float32, 0.1),
}
# the tensors of cfg3 and cfg4 read as rows of scalars: one feature per head (bench.py --scalar-heads); compared whole
ONE_FEATURE_HEADS = {
    "cfg3_heads1": (128, 4096, 128, 128, 16, 3, torch.bfloat16, 1.0),
    "cfg4_heads1": (128, 8192, 128, 128, 2, 13, torch.float32, 1.0),
}
ALL_CONFIGS = {**CONFIGS, **ONE_FEATURE_HEADS}


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import ncn_cuda_module
    return ncn_cuda_module


def _inputs(name):
    batch, N, E, C, n, L, dtype, wscale = ALL_CONFIGS[name]
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(batch, N, E, device="cuda", generator=g).to(dtype)
    xa = (0.5 * torch.randn(batch, N, E, device="cuda", generator=g)).to(dtype)
    dy = torch.randn(batch, N, E, device="cuda", generator=g).to(dtype)
    W = (torch.randn(L, 2 * E, device="cuda", generator=g) * wscale / n ** 0.5).to(dtype).float()
    return x, xa, dy, W


def _segment(n, L=None, elements=None):
    """Stages per saved checkpoint, as bench.py and the whole-net autograd node choose it."""
    from ncn_cuda_amd.modules import default_save_every
    return default_save_every(n, L, elements)


def _run(M, x, xa, dy, W, C, n, L, dtype, want_inputs=False, with_inputs=False):
    """Forward + reversible backward the way bench.py's timed step and the autograd nodes run the configuration:
    segments of default_save_every(n) stages, and no reconstructed inputs asked of the backward (want_inputs=False: the
    state between the stages of a segment travels through the workspace and the last pass writes gradients only).
    want_inputs=True is the other form of the call, which also returns the reconstructed inputs of every segment."""
    seg = _segment(n, L, x.numel())
    saved, spans = [], []
    cx, cxa = x, xa
    for a in range(0, L, seg):
        cnt = min(seg, L - a)
        if cnt == 1:     # bf16: the outputs are saved with what their rounding took away (two bf16 planes)
            cx, cxa, sy, sya = M.forward_stages_saving(cx, cxa, W[a], 0.9, 0, n, C, a)
            saved.append((sy, sya))
        else:
            cx, cxa = M.forward_stages(cx, cxa, W[a:a + cnt], 0.9, 0, n, C, a, cnt, out_dtype=torch.float32)
            saved.append((cx, cxa))
        spans.append((a, cnt))
    g, h = dy, None
    dWs = [None] * len(spans)
    xr = xar = None
    for k in range(len(spans) - 1, -1, -1):
        a, cnt = spans[k]
        xr, xar, g, h, dWs[k] = M.backward_stages(saved[k][0], saved[k][1], g, h, W[a:a + cnt], 0.9, 0, n, C, a, cnt,
                                                  grad_dtype=dtype if cnt == 1 else torch.float32,
                                                  want_inputs=want_inputs)
    if with_inputs:
        return cx, cxa, g, h, torch.cat(dWs), xr, xar
    return cx, cxa, g, h, torch.cat(dWs)


@pytest.mark.parametrize("name", ["cfg2", "cfg4", "cfg5"])
def test_full_size_with_and_without_reconstructed_inputs(M, name):
    """The two forms of the backward call at full size: the one that is timed (no reconstructed inputs) and the one
    that also writes them.  They run the same kernels on the same values, so the gradients must agree bit for bit; the
    reconstructed inputs of the first segment are the network inputs, to the rounding that reversing
    default_save_every(n) stages amplifies."""
    batch, N, E, C, n, L, dtype, _ = CONFIGS[name]
    x, xa, dy, W = _inputs(name)
    timed = _run(M, x, xa, dy, W, C, n, L, dtype)
    other = _run(M, x, xa, dy, W, C, n, L, dtype, want_inputs=True, with_inputs=True)
    for a, b in zip(timed, other[:5]):
        assert torch.equal(a, b)
    amp = (1 / 0.9) ** (n * min(_segment(n, L, x.numel()), L))
    errs = {"x_rec": O.rel_err(other[5], x.float()), "xa_rec": O.rel_err(other[6], xa.float())}
    print(f"measured reconstruction errors {name} (want_inputs=True): " + json.dumps(errs))
    if os.environ.get("NCN_ERROR_REPORT"):
        with open(os.environ["NCN_ERROR_REPORT"], "a") as fh:
            fh.write(json.dumps({"config": name, "form": "want_inputs", **errs}) + "\n")
    for v in errs.values():
        assert v < max(1e-5, 1e-6 * amp)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size_slice_parity_and_dw_additivity(M, name):
    batch, N, E, C, n, L, dtype, _ = CONFIGS[name]
    x, xa, dy, W = _inputs(name)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    y, ya, dx, dxa, dW = _run(M, x, xa, dy, W, C, n, L, dtype)
    again = _run(M, x, xa, dy, W, C, n, L, dtype)
    for a, b in zip((y, ya, dx, dxa, dW), again):
        assert torch.equal(a, b)                                   # deterministic, dW included
    # the first two batch entries against the oracle (float64 on the same stored values)
    k = 2
    d = torch.float64
    ref = O.net_autograd(x[:k].cpu().to(d), xa[:k].cpu().to(d), [w.cpu().to(d) for w in W], dy[:k].cpu().to(d),
                         torch.zeros(k, N, E, dtype=d), 0.9, n, C)
    gtol = tol                                                     # float32: 1e-5 on the gradients too
    assert O.rel_err(y[:k], ref[0]) < tol and O.rel_err(ya[:k], ref[1]) < tol
    assert O.rel_err(dx[:k], ref[2]) < gtol and O.rel_err(dxa[:k], ref[3]) < gtol
    # dW of the two entries alone (GPU) against the oracle, then additivity over batch chunks for the rest
    part = _run(M, x[:k].contiguous(), xa[:k].contiguous(), dy[:k].contiguous(), W, C, n, L, dtype)[4]
    for l in range(L):
        assert O.rel_err(part[l], ref[4][l]) < gtol
    chunks = 4
    step = batch // chunks
    total = torch.zeros_like(dW, dtype=torch.float64)
    for c in range(chunks):
        s = slice(c * step, (c + 1) * step)
        total += _run(M, x[s].contiguous(), xa[s].contiguous(), dy[s].contiguous(), W, C, n, L, dtype)[4].double()
    assert O.rel_err(dW, total) < 1e-5                             # float32 sums in a different order


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size_inverse_round_trip(M, name):
    """inverse(forward(x, xa)) == (x, xa); the target for the reconstruction of configuration 5 is 1e-4."""
    batch, N, E, C, n, L, dtype, _ = CONFIGS[name]
    x, xa, _, W = _inputs(name)
    x, xa = x.float(), xa.float()
    seg = _segment(n, L, x.numel())
    for a in range(0, L, seg):            # reversal is only asked over what one saved checkpoint covers
        cnt = min(seg, L - a)
        y, ya = M.forward_stages(x, xa, W[a:a + cnt], 0.9, 0, n, C, a, cnt)
        xi, xai = M.inverse_stages(y, ya, W[a:a + cnt], 0.9, 0, n, C, a, cnt)
        assert O.rel_err(xi, x) < 1e-4 and O.rel_err(xai, xa) < 1e-4
        x, xa = y, ya


@pytest.mark.parametrize("case", [
    (4100, 4096, 128, 4, 16, 1, 1, torch.bfloat16),   # one-stage register kernels, 2.15e9 elements per array
    (2060, 8192, 128, 4, 2, 0, 6, torch.float32),     # multi-stage passes, 2.16e9 elements per array
], ids=["n16_bf16_one_stage", "n2_f32_six_stages"])
def test_more_than_2_31_elements_per_array(M, case):
    """Arrays past 2^31 elements (a 288 GB card holds them): element offsets must be 64-bit all the way.  Batch entries
    are independent, so the first, middle and last entries are checked against the oracle on just those entries, and dW
    against the sum of the dW of the two halves of the batch."""
    batch, N, E, C, n, stage, L, dtype = case
    assert batch * N * E > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.empty(batch, N, E, device="cuda", dtype=dtype).normal_(generator=g)
    xa = torch.empty(batch, N, E, device="cuda", dtype=dtype).normal_(generator=g)
    dy = torch.empty(batch, N, E, device="cuda", dtype=dtype).normal_(generator=g)
    W = torch.randn(L, 2 * E, device="cuda", generator=g) * (0.5 / n ** 0.5)
    if L > 1:
        y, ya = M.forward_stages(x, xa, W, 0.9, 0, n, C, stage, L)
        sy, sya, gd = y, ya, torch.float32
    else:
        y, ya, sy, sya = M.forward_stages_saving(x, xa, W[0], 0.9, 0, n, C, stage)
        gd = dtype
    Wc = W if L > 1 else W[0]
    xr, xar, dx, dxa, dW = M.backward_stages(sy, sya, dy, None, Wc, 0.9, 0, n, C, stage, L, grad_dtype=gd)
    sel = [0, batch // 2, batch - 2, batch - 1]
    f = torch.float64
    xs, xas, dys = x[sel].cpu().to(f), xa[sel].cpu().to(f), dy[sel].cpu().to(f)
    ref = O.net_autograd(xs, xas, [w.cpu().to(f) for w in W], dys, torch.zeros_like(dys), 0.9, n, C, first_stage=stage)
    tol = 2e-2 if dtype == torch.bfloat16 else max(1e-5, 2e-6 * (1 / 0.9) ** (n * L))
    for got, want in ((y, ref[0]), (ya, ref[1]), (dx, ref[2]), (dxa, ref[3]), (xr, xs), (xar, xas)):
        assert O.rel_err(got[sel].float().cpu(), want) < tol
    del x, xa, y, ya, dx, dxa, xr, xar
    torch.cuda.empty_cache()
    h = batch // 2
    cut = lambda t, sl: (t[:, sl] if t.dim() == 4 else t[sl]).contiguous()     # saved outputs may be [2, batch, N, E]
    halves = [M.backward_stages(cut(sy, sl), cut(sya, sl), dy[sl].contiguous(), None, Wc, 0.9, 0, n, C,
                                stage, L, grad_dtype=gd)[4] for sl in (slice(0, h), slice(h, batch))]
    assert O.rel_err(dW, halves[0] + halves[1]) < 1e-4
    del sy, sya, dy, halves
    torch.cuda.empty_cache()


@pytest.mark.parametrize("name,entries", [("cfg2", None), ("cfg5", None), ("cfg3", None), ("cfg4", None),
                                          ("cfg3_heads1", None), ("cfg4_heads1", 16)])
def test_whole_tensor_against_the_c_oracle(M, name, entries):
    """Every element, not a slice: the configuration as bench.py's timed step runs it (backward without reconstructed
    inputs) against the plain C restatement in float64
    (oracle/ncn_oracle.c on the host threads: about 25 s for the four configurations on 16 threads).  `entries` cuts
    the comparison to that many batch entries spread over the batch, for a machine where that is too long."""
    from oracle import c_oracle as CO
    batch, N, E, C, n, L, dtype, _ = ALL_CONFIGS[name]
    x, xa, dy, W = _inputs(name)
    y, ya, dx, dxa, dW = _run(M, x, xa, dy, W, C, n, L, dtype)
    sel = list(range(batch)) if entries is None else sorted({(k * batch) // entries for k in range(entries)} | {batch - 1})
    d = torch.float64
    ref = CO.net_forward_backward(x[sel].cpu().to(d), xa[sel].cpu().to(d), [w.cpu().to(d) for w in W], dy[sel].cpu().to(d),
                                  None, 0.9, n, C, keep_outputs=False)   # float64: reversal costs nothing, L copies do
    # 2e-2 with bf16 storage, 1e-5 in float32, for the outputs and for every gradient (max |diff| / max |ref| over the
    # whole tensor; the root-mean-square figure is recorded beside it)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    got = {"y": y[sel], "ya": ya[sel], "dx": dx[sel], "dxa": dxa[sel]}
    want = {"y": ref[0], "ya": ref[1], "dx": ref[2], "dxa": ref[3]}
    report = {k: {"max": O.rel_err(got[k].float().cpu(), want[k]), "rms": O.rms_err(got[k].float().cpu(), want[k])}
              for k in got}
    if entries is None:                                            # dW sums over the whole batch
        per_stage = [O.rel_err(dW[l].cpu(), ref[4][l]) for l in range(L)]
        report["dW_worst"] = {"max": max(per_stage), "rms": max(O.rms_err(dW[l].cpu(), ref[4][l]) for l in range(L))}
    print(f"measured errors {name} (segments of {_segment(n, L, x.numel())} stages): " + json.dumps(report))
    if os.environ.get("NCN_ERROR_REPORT"):                         # a file to read the figures from after a run
        with open(os.environ["NCN_ERROR_REPORT"], "a") as fh:
            fh.write(json.dumps({"config": name, "segment": _segment(n, L, x.numel()), **report}) + "\n")
    for k, v in report.items():
        assert v["max"] < tol, (k, v)


def test_headline_shape_with_table_and_lengths_against_the_c_oracle(M):
    """cfg3 through the table / context-length entry points (a different length per batch entry, a radix-16 table on
    stage 1), every element against the C oracle in float64."""
    from oracle import c_oracle as CO
    batch, N, E, C, n, L, dtype, _ = CONFIGS["cfg3"]
    x, xa, dy, W = _inputs("cfg3")
    tables = [O.stride_group_table(N, n, 0), O.radix_group_table(N, n, 1), O.stride_group_table(N, n, 2)]
    lens = (N - 1 - 37 * torch.arange(batch)) % (N + 1)
    lens[0], lens[1] = N, 0
    gt = [t.to(torch.int32).cuda() for t in tables]
    gl = lens.to(torch.int32).cuda()
    saved, cx, cxa = [], x, xa
    for l in range(L):
        cx, cxa, sy, sya = M.forward_stages_saving(cx, cxa, W[l], 0.9, 0, n, C, l, group_index=gt[l], ctx_len=gl)
        saved.append((sy, sya))
    g, h, dWs = dy, None, [None] * L
    for l in range(L - 1, -1, -1):
        _, _, g, h, dWs[l] = M.backward_stages(saved[l][0], saved[l][1], g, h, W[l], 0.9, 0, n, C, l, 1, grad_dtype=dtype,
                                               want_inputs=False, group_index=gt[l], ctx_len=gl)
    d = torch.float64
    ref = CO.net_forward_backward(x.cpu().to(d), xa.cpu().to(d), [w.cpu().to(d) for w in W], dy.cpu().to(d), None, 0.9, n,
                                  C, tables=tables, ctx_len=lens)
    tol = 2e-2
    assert O.rel_err(cx.float().cpu(), ref[0]) < tol and O.rel_err(cxa.float().cpu(), ref[1]) < tol
    assert O.rel_err(g.float().cpu(), ref[2]) < tol and O.rel_err(h.float().cpu(), ref[3]) < tol
    for l in range(L):
        assert O.rel_err(dWs[l][0].cpu(), ref[4][l]) < tol, l


def test_deep_shape_with_lengths_against_the_c_oracle(M):
    """cfg4 with one context length per batch entry and no table: the multi-stage passes for groups of two rows in their
    LENGTHS build (13 stages in two passes forward, three backward), every element against the C oracle in float64 on
    the stride tables with the same lengths."""
    from oracle import c_oracle as CO
    batch, N, E, C, n, L, dtype, _ = CONFIGS["cfg4"]
    x, xa, dy, W = _inputs("cfg4")
    lens = (N - 1 - 61 * torch.arange(batch)) % (N + 1)
    lens[0], lens[1], lens[2] = N, 0, 1
    gl = lens.to(torch.int32).cuda()
    y, ya = M.forward_stages(x, xa, W, 0.9, 0, n, C, 0, L, ctx_len=gl)
    xr, xar, dx, dxa, dW = M.backward_stages(y, ya, dy, None, W, 0.9, 0, n, C, 0, L, ctx_len=gl)
    tables = [O.stride_group_table(N, n, l) for l in range(L)]
    d = torch.float64
    ref = CO.net_forward_backward(x.cpu().to(d), xa.cpu().to(d), [w.cpu().to(d) for w in W], dy.cpu().to(d), None, 0.9, n,
                                  C, tables=tables, ctx_len=lens, keep_outputs=False)
    errs = {"y": O.rel_err(y.cpu(), ref[0]), "ya": O.rel_err(ya.cpu(), ref[1]), "dx": O.rel_err(dx.cpu(), ref[2]),
            "dxa": O.rel_err(dxa.cpu(), ref[3]), "x_rec": O.rel_err(xr.cpu(), x.cpu().to(d)),
            "dW_worst": max(O.rel_err(dW[l].cpu(), ref[4][l]) for l in range(L))}
    print("measured errors cfg4 with lengths: " + json.dumps(errs))
    for k, v in errs.items():
        assert v < 1e-5, (k, v)


def test_deep_shape_radix_levels_against_the_c_oracle(M):
    """cfg4's tensors through the 13 levels of the radix-2 grouping (two multi-level LDS passes each way), every element
    against the C oracle in float64 on the radix tables."""
    from oracle import c_oracle as CO
    batch, N, E, C, n, L, dtype, _ = CONFIGS["cfg4"]
    x, xa, dy, W = _inputs("cfg4")
    y, ya = M.forward_radix(x, xa, W, 0.9, 0, n, C, 0, L)
    xr, xar, dx, dxa, dW = M.backward_radix(y, ya, dy, None, W, 0.9, 0, n, C, 0, L)
    tables = [O.radix_group_table(N, n, l) for l in range(L)]
    d = torch.float64
    ref = CO.net_forward_backward(x.cpu().to(d), xa.cpu().to(d), [w.cpu().to(d) for w in W], dy.cpu().to(d), None, 0.9, n,
                                  C, tables=tables, keep_outputs=False)
    gtol = max(1e-5, 3e-6 * (1 / 0.9) ** (n * L))
    assert O.rel_err(y.cpu(), ref[0]) < 1e-5 and O.rel_err(ya.cpu(), ref[1]) < 1e-5
    assert O.rel_err(dx.cpu(), ref[2]) < gtol and O.rel_err(dxa.cpu(), ref[3]) < gtol
    assert O.rel_err(xr.cpu(), x.cpu().to(d)) < gtol
    for l in range(L):
        assert O.rel_err(dW[l].cpu(), ref[4][l]) < gtol, l
