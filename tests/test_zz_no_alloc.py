"""ncn_backward_static: the backward without workspace argument or allocation, against ncn_backward.

Two calls in a row through the C ABI, the second on a smaller problem: the library's own scratch keeps what the first
call left there, and nothing of it may leak into the second result."""
import ctypes

import pytest
import torch

from oracle import ncn_oracle as O

pytestmark = pytest.mark.gpu


def _call_both(lib, _lib, shape5, n_stages, seed, dtype=torch.float32):
    batch, N, E, C, n = shape5
    x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, n_stages, n, seed=seed, xa_zero=False)
    dev = torch.device("cuda:0")
    W = torch.stack(Ws).to(dev)
    sh = _lib.NcnShape(batch, N, E, C, n)
    f32 = torch.float32
    # outputs of the stages: the saved tensors a backward starts from (float32, as the autograd node keeps them)
    y, ya = x.to(dev), xa.to(dev)
    for l in range(n_stages):
        y2, ya2 = torch.empty_like(y), torch.empty_like(ya)
        rc = lib.ncn_forward(y.data_ptr(), ya.data_ptr(), 0, y2.data_ptr(), ya2.data_ptr(), 0, None, None,
                             W[l].data_ptr(), None, 0, ctypes.byref(sh), l, 1, 0.9, 0.9, 0, None)
        assert rc == 0
        y, ya = y2, ya2
    gdy, gdya = dy.to(dev).to(dtype), dya.to(dev).to(dtype)
    code = 0 if dtype == f32 else 1
    gcode = code if n_stages == 1 else 0

    def outputs():
        gd = dtype if n_stages == 1 else f32
        return (torch.full((batch, N, E), float("nan"), device=dev, dtype=gd), torch.full((batch, N, E), float("nan"), device=dev, dtype=gd),
                torch.full((batch, N, E), float("nan"), device=dev), torch.full((batch, N, E), float("nan"), device=dev),
                torch.full((n_stages, 2 * E), float("nan"), device=dev))

    ws_bytes = lib.ncn_workspace_bytes(ctypes.byref(sh))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    a = outputs()
    rc = lib.ncn_backward(y.data_ptr(), ya.data_ptr(), 0, gdy.data_ptr(), gdya.data_ptr(), code, a[0].data_ptr(), a[1].data_ptr(),
                          gcode, a[2].data_ptr(), a[3].data_ptr(), W.data_ptr(), a[4].data_ptr(), ws.data_ptr(),
                          ctypes.c_size_t(ws_bytes), ctypes.byref(sh), 0, n_stages, 0.9, 0.9, 0, None)
    assert rc == 0, _lib.error_string(rc)
    b = outputs()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.ncn_backward_static(y.data_ptr(), ya.data_ptr(), 0, gdy.data_ptr(), gdya.data_ptr(), code, b[0].data_ptr(),
                                 b[1].data_ptr(), gcode, b[2].data_ptr(), b[3].data_ptr(), W.data_ptr(), b[4].data_ptr(),
                                 ctypes.byref(sh), 0, n_stages, 0.9, 0.9, 0, None)
    assert rc == 0, _lib.error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return a, b


def test_backward_static_matches_backward_on_two_calls_in_a_row():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import _lib
    lib = _lib.load()
    assert 0 < lib.ncn_static_scratch_bytes() <= 16 << 20
    # first call: more wave tiles (40 * 128 = 5120) than the scratch has partial rows (4096): the grid is capped at
    # 4096 partial rows and its waves loop over tiles, where ncn_backward launches a wave per tile; bf16 gradients
    a, b = _call_both(lib, _lib, (40, 4096, 128, 4, 16), 1, seed=3, dtype=torch.bfloat16)
    for u, v in zip(a[:4], b[:4]):
        assert torch.equal(u, v)                         # dx, dxa, x_rec, xa_rec do not depend on the grid
    assert O.rel_err(b[4], a[4]) < 1e-5 and torch.isfinite(b[4]).all()   # the same terms summed over fewer partial rows
    # the capped grid is rounded to whole multiples of n_head waves: three heads (blocks in threes) and two
    # (and one feature per head: 16 lanes' worth of heads, waves in sixteens)
    for shape5 in ((40, 4096, 96, 3, 16), (40, 4096, 64, 2, 16), (40, 4096, 64, 64, 16)):
        a, b = _call_both(lib, _lib, shape5, 1, seed=6)
        for u, v in zip(a[:4], b[:4]):
            assert torch.equal(u, v)
        assert O.rel_err(b[4], a[4]) < 1e-5 and torch.isfinite(b[4]).all()
    # second call, smaller, three stages: what the first call left in the scratch must not show
    a, b = _call_both(lib, _lib, (2, 96, 32, 4, 4), 3, seed=4)
    for u, v in zip(a, b):
        assert torch.isfinite(v).all() and O.rel_err(v, u) < 1e-5
    # generic kernels (n_cache = 3) use the scratch too
    a, b = _call_both(lib, _lib, (2, 36, 20, 2, 3), 1, seed=5)
    for u, v in zip(a, b):
        assert torch.isfinite(v).all() and O.rel_err(v, u) < 1e-5


def test_backward_static_rejects_what_its_scratch_cannot_hold():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import _lib
    lib = _lib.load()
    sh = _lib.NcnShape(1, 16, 512, 4, 4)                  # E = 512: a partial row of 1024 floats
    p = ctypes.c_void_p(4096)                             # never dereferenced: the size check comes first
    rc = lib.ncn_backward_static(p, p, 0, p, p, 0, p, p, 0, None, None, p, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, None)
    assert rc == -9 and "scratch" in _lib.error_string(rc)


def test_backward_static_needs_the_state_buffers_for_several_stages():
    """With n_stages > 1 the stages hand their reconstructed inputs on through x_rec, xa_rec; ncn_backward takes two
    arrays from its workspace when they are NULL, the static scratch has no room for them: NCN_ERR_ALIAS."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import _lib
    lib = _lib.load()
    batch, N, E, C, n, L = 2, 64, 32, 4, 4, 3
    dev = torch.device("cuda:0")
    sh = _lib.NcnShape(batch, N, E, C, n)
    t = [torch.randn(batch, N, E, device=dev) for _ in range(3)]
    out = [torch.empty(batch, N, E, device=dev) for _ in range(2)]
    W = torch.randn(L, 2 * E, device=dev) * 0.3
    dW = torch.empty(L, 2 * E, device=dev)
    rc = lib.ncn_backward_static(t[0].data_ptr(), t[1].data_ptr(), 0, t[2].data_ptr(), None, 0, out[0].data_ptr(),
                                 out[1].data_ptr(), 0, None, None, W.data_ptr(), dW.data_ptr(), ctypes.byref(sh), 0, L,
                                 0.9, 0.9, 0, None)
    assert rc == -8 and "x_rec" in _lib.error_string(rc)
    # one stage takes the NULLs, as ncn_backward does
    rc = lib.ncn_backward_static(t[0].data_ptr(), t[1].data_ptr(), 0, t[2].data_ptr(), None, 0, out[0].data_ptr(),
                                 out[1].data_ptr(), 0, None, None, W.data_ptr(), dW.data_ptr(), ctypes.byref(sh), 0, 1,
                                 0.9, 0.9, 0, None)
    torch.cuda.synchronize()
    assert rc == 0 and torch.isfinite(out[0]).all() and torch.isfinite(dW[0]).all()


def test_backward_static_under_graph_capture():
    """What the entry point is for: after one warm-up call (which resolves the scratch's address and is not
    capturable), a call recorded into a HIP graph replays on new inputs like the eager ncn_backward."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ncn_cuda_amd import _lib
    lib = _lib.load()
    batch, N, E, C, n = 4, 256, 128, 4, 16
    dev = torch.device("cuda:0")
    sh = _lib.NcnShape(batch, N, E, C, n)
    sets = [O.make_inputs(batch, N, E, 1, n, seed=70 + k, xa_zero=False) for k in range(3)]
    W = sets[0][2][0].to(dev)
    y, ya, dy, dya = (torch.empty(batch, N, E, device=dev) for _ in range(4))
    dx, dxa = torch.empty_like(y), torch.empty_like(y)
    dW = torch.empty(1, 2 * E, device=dev)

    def load(k):   # the stage outputs of input set k, and its upstream gradients
        x, xa = sets[k][0].to(dev), sets[k][1].to(dev)
        rc = lib.ncn_forward(x.data_ptr(), xa.data_ptr(), 0, y.data_ptr(), ya.data_ptr(), 0, None, None, W.data_ptr(), None, 0,
                             ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, None)
        assert rc == 0
        dy.copy_(sets[k][3]); dya.copy_(sets[k][4])

    def static_call(stream):
        return lib.ncn_backward_static(y.data_ptr(), ya.data_ptr(), 0, dy.data_ptr(), dya.data_ptr(), 0, dx.data_ptr(),
                                       dxa.data_ptr(), 0, None, None, W.data_ptr(), dW.data_ptr(), ctypes.byref(sh), 0, 1,
                                       0.9, 0.9, 0, stream)

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert static_call(ctypes.c_void_p(side.cuda_stream)) == 0      # warm-up, outside any capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        before = torch.cuda.memory_allocated()
        assert static_call(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        assert torch.cuda.memory_allocated() == before
    ws_bytes = lib.ncn_workspace_bytes(ctypes.byref(sh))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    for k in (1, 2, 0, 1):
        load(k)
        dx.fill_(float("nan")); dxa.fill_(float("nan")); dW.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [dx.clone(), dxa.clone(), dW.clone()]
        ex, exa, eW = torch.empty_like(dx), torch.empty_like(dx), torch.empty_like(dW)    # eager work between the replays
        rc = lib.ncn_backward(y.data_ptr(), ya.data_ptr(), 0, dy.data_ptr(), dya.data_ptr(), 0, ex.data_ptr(), exa.data_ptr(), 0,
                              None, None, W.data_ptr(), eW.data_ptr(), ws.data_ptr(), ctypes.c_size_t(ws_bytes),
                              ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(got[0], ex) and torch.equal(got[1], exa)
        assert O.rel_err(got[2], eW) < 1e-5 and torch.isfinite(got[2]).all()
