"""The library under HIP graph capture: it launches on the stream it is given, never synchronises, allocates or
clears memory, so a forward + backward step can be captured once and replayed.  Every replay is checked against the
same step run eagerly, with eager work and synchronisations between the replays."""
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


def _step(M, x, xa, W, dy, alpha, n, C, L, per_stage):
    """Forward of L stages and reversible backward; per_stage: one call per stage (outputs saved per stage), else one
    call for the whole segment (multi-stage passes where the shape allows)."""
    if per_stage:
        saved = []
        cx, cxa = x, xa
        for l in range(L):
            cx, cxa, y32, ya32 = M.forward_stages(cx, cxa, W[l], alpha, 0, n, C, l, 1, save_fp32=True)
            saved.append((y32, ya32))
        g, h = dy, None
        dWs = []
        for l in range(L - 1, -1, -1):
            _, _, g, h, dW = M.backward_stages(saved[l][0], saved[l][1], g, h, W[l], alpha, 0, n, C, l, 1,
                                               want_inputs=False)
            dWs.append(dW)
        return cx, cxa, g, h, torch.cat(dWs[::-1])
    y, ya = M.forward_stages(x, xa, W, alpha, 0, n, C, 0, L, out_dtype=torch.float32)
    _, _, g, h, dW = M.backward_stages(y, ya, dy, None, W, alpha, 0, n, C, 0, L, grad_dtype=torch.float32)
    return y, ya, g, h, dW


@pytest.mark.parametrize("case", [(4, 256, 128, 4, 16, 3, torch.bfloat16, True), (4, 512, 64, 2, 2, 8, torch.float32, False)],
                         ids=["per_stage_n16_bf16", "multi_stage_n2_f32"])
def test_capture_and_replay_matches_eager(M, case):
    batch, N, E, C, n, L, dtype, per_stage = case
    alpha = 0.9
    inputs = [O.make_inputs(batch, N, E, L, n, seed=50 + k, xa_zero=False, dtype=dtype) for k in range(3)]
    W = torch.stack([w.float() for w in inputs[0][2]]).cuda()
    sx = torch.empty(batch, N, E, dtype=dtype, device="cuda")
    sxa, sdy = torch.empty_like(sx), torch.empty_like(sx)

    def load(k):
        sx.copy_(inputs[k][0]); sxa.copy_(inputs[k][1]); sdy.copy_(inputs[k][3])

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # warm-up on the side stream, as graph capture wants
        for _ in range(2):
            _step(M, sx, sxa, W, sdy, alpha, n, C, L, per_stage)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _step(M, sx, sxa, W, sdy, alpha, n, C, L, per_stage)
    for k in (1, 2, 0, 1):
        load(k)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        eager = _step(M, sx, sxa, W, sdy, alpha, n, C, L, per_stage)   # eager work between replays
        torch.cuda.synchronize()
        for a, b in zip(got, eager):
            assert torch.equal(a, b)
    # and the replayed numbers are the right ones
    f = torch.float32
    x, xa, _, dy, _ = inputs[1]
    Ws = inputs[0][2]                      # the weights were fixed before the capture
    ref = O.net_autograd(x.to(f).double(), xa.to(f).double(), [w.to(f).double() for w in Ws], dy.to(f).double(),
                         torch.zeros(batch, N, E, dtype=torch.float64), alpha, n, C)
    tol = 2e-2 if dtype == torch.bfloat16 else 3e-5
    assert O.rel_err(got[0], ref[0]) < tol and O.rel_err(got[2], ref[2]) < tol
    assert O.rel_err(got[4].reshape(L, -1)[0], ref[4][0]) < tol
