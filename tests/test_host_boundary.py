"""The C-ABI library and the host-side argument checks, without a GPU: the shared object loads, exports every
function include/ncn_hip.h declares, and rejects bad arguments before any GPU work."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "ncn_hip.h")


@pytest.fixture(scope="module")
def lib():
    from ncn_cuda_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from ncn_cuda_amd import _build
        _build.build()
    return _lib


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ncn_[a-z_0-9]+)\s*\(", text)))


def test_header_functions_are_exported(lib):
    names = _declared_functions()
    assert {"ncn_forward", "ncn_backward", "ncn_inverse", "ncn_workspace_bytes", "ncn_workspace_bytes_stages",
            "ncn_plan_passes", "ncn_kernel_path",
            "ncn_check_shape", "ncn_error_string", "ncn_version"} <= set(names)
    handle = lib.load()
    for name in names:
        assert getattr(handle, name) is not None, name
    assert sorted(lib.EXPORTS) == names
    assert re.fullmatch(r"\d+\.\d+", handle.ncn_version().decode())


def _shape(lib, batch, N, E, C, n):
    return lib.NcnShape(batch, N, E, C, n)


def test_check_shape_codes(lib):
    h = lib.load()
    ok = _shape(lib, 2, 64, 32, 4, 4)
    assert h.ncn_check_shape(ctypes.byref(ok), 0, 1, 0) == 0
    assert h.ncn_check_shape(None, 0, 1, 0) == -1
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 2, 65, 32, 4, 4)), 0, 1, 0) == -2   # N % n_cache
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 2, 64, 30, 4, 4)), 0, 1, 0) == -2   # E % n_head
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 0, 64, 32, 4, 4)), 0, 1, 0) == -2
    assert h.ncn_check_shape(ctypes.byref(ok), -1, 1, 0) == -2
    assert h.ncn_check_shape(ctypes.byref(ok), 0, 0, 0) == -2
    assert h.ncn_check_shape(ctypes.byref(ok), 0, 1, 7) == -4                             # activation
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 1, 256, 32, 4, 128)), 0, 1, 0) == -6  # n_cache > 64
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 1, 64, 512, 4, 4)), 0, 1, 0) == 0     # head width 128: register kernel
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 1, 64, 512, 4, 4)), 0, 1, 1) == 0     # .. with relu too
    assert h.ncn_check_shape(ctypes.byref(_shape(lib, 1, 64, 1024, 4, 4)), 0, 1, 0) == -6   # head width 256
    for code in (0, -1, -2, -3, -4, -5, -6, -7, -8):
        assert len(h.ncn_error_string(code)) > 0


def test_kernel_path_and_workspace(lib):
    h = lib.load()
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 128, 4096, 128, 4, 16))) == 2   # headline shape: register kernels
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 1, 256, 32, 4, 2))) == 2        # config 1 (Ec = 8)
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 1, 24, 10, 2, 3))) == 1         # n = 3, Ec = 5: generic
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 1, 256, 32, 4, 128))) == 0
    # one feature per head: register kernels (four heads to a lane) when E is a multiple of 4 and n_cache a power of two
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 2, 256, 128, 128, 16))) == 2
    assert h.ncn_kernel_path_scalars(ctypes.byref(_shape(lib, 2, 256, 128, 128, 16)), 1e-4, 0.9) == 1
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 2, 256, 6, 6, 16))) == 1
    assert h.ncn_kernel_path(ctypes.byref(_shape(lib, 2, 240, 128, 128, 3))) == 1
    ws = h.ncn_workspace_bytes(ctypes.byref(_shape(lib, 128, 4096, 128, 4, 16)))
    assert ws > 0 and ws % 16 == 0 and ws < (1 << 25)
    assert h.ncn_workspace_bytes(ctypes.byref(_shape(lib, 1, 65, 32, 4, 4))) == 0
    # multi-stage passes: deep small-group stacks ask for ping-pong arrays, the headline shape (n_cache = 16) does not
    deep = _shape(lib, 128, 8192, 128, 4, 2)
    P4 = 128 * 8192 * 128 * 4
    assert h.ncn_workspace_bytes_stages(ctypes.byref(deep), 0, 13, 0, 0) == 2 * P4
    # backward: the four arrays and a dW partial row per window and stage of every pass (stages 6-12 in 4096 closed
    # windows per head, stages 3-5 in 128 x 4 x 9 halo windows that own 114 of their 128 groups, stages 0-2 in 128 x 34
    # that own 122), plus their chunk sums (one row per 32, + 8)
    rows = 7 * 4096 + 3 * 4608 + 3 * 4352
    assert h.ncn_workspace_bytes_stages(ctypes.byref(deep), 0, 13, 0, 1) == (rows + rows // 32 + 8) * 2 * 128 * 4 + 4 * P4
    assert (rows + rows // 32 + 8) * 2 * 128 * 4 > h.ncn_workspace_bytes(ctypes.byref(deep))
    assert h.ncn_workspace_bytes_stages(ctypes.byref(deep), 0, 1, 0, 0) == 0
    head = _shape(lib, 128, 4096, 128, 4, 16)
    assert h.ncn_workspace_bytes_stages(ctypes.byref(head), 0, 3, 0, 1) == h.ncn_workspace_bytes(ctypes.byref(head))
    # scalars the register kernels' scaled state cannot carry go to the generic kernels, or nowhere for wide heads
    for alpha, m, want in ((0.9, 0.9, 2), (1e-4, 0.9, 1), (0.9, 0.9995, 1), (0.9, 5e-4, 1), (40.0, 0.9, 2), (2000.0, 0.9, 1), (1e-3, 0.999, 2)):
        assert h.ncn_kernel_path_scalars(ctypes.byref(head), alpha, m) == want, (alpha, m)
    wide = _shape(lib, 2, 64, 256, 2, 8)        # heads of 128: register kernels only
    assert h.ncn_kernel_path_scalars(ctypes.byref(wide), 0.9, 0.9) == 2
    assert h.ncn_kernel_path_scalars(ctypes.byref(wide), 1e-4, 0.9) == 0


def test_entry_points_reject_bad_arguments_before_touching_the_gpu(lib):
    h = lib.load()
    sh = _shape(lib, 2, 64, 32, 4, 4)
    p = ctypes.c_void_p(4096)       # never dereferenced: every call below fails validation first
    z = ctypes.c_void_p(0)
    odd = ctypes.c_void_p(4100)
    nows = (z, ctypes.c_size_t(0))
    assert h.ncn_forward(z, p, 0, p, p, 0, z, z, p, *nows, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -1
    assert h.ncn_forward(p, p, 5, p, p, 0, z, z, p, *nows, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -3
    assert h.ncn_forward(odd, p, 0, p, p, 0, z, z, p, *nows, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -7
    assert h.ncn_forward(p, p, 0, p, p, 0, p, z, p, *nows, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -1  # y32 without ya32
    assert h.ncn_inverse(p, p, 0, z, p, 0, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -1
    ws = h.ncn_workspace_bytes(ctypes.byref(sh))
    args = [p, p, 0, p, p, 0, p, p, 0, z, z, p, p]
    assert h.ncn_backward(*args, z, ctypes.c_size_t(0), ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -5
    assert h.ncn_backward(*args, p, ctypes.c_size_t(ws - 1), ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -5
    # two stages without x_rec, xa_rec and without room in the workspace for the state between them (groups of 8 rows:
    # one launch per stage; shapes with multi-stage passes may run two stages as one closed pass, which carries nothing)
    sh8 = _shape(lib, 2, 64, 32, 4, 8)
    ws8 = h.ncn_workspace_bytes(ctypes.byref(sh8))
    assert h.ncn_backward(*args, p, ctypes.c_size_t(ws8), ctypes.byref(sh8), 0, 2, 0.9, 0.9, 0, z) == -8  # needs x_rec


def test_indexed_entry_points_reject_bad_arguments_before_touching_the_gpu(lib):
    h = lib.load()
    sh = _shape(lib, 2, 64, 32, 4, 4)
    p = ctypes.c_void_p(4096)       # never dereferenced: every call below fails validation first
    z = ctypes.c_void_p(0)
    odd4 = ctypes.c_void_p(4098)    # an int32 table must be 4-byte aligned
    fwd = lambda x, table, lens, act=0: h.ncn_forward_indexed(x, p, 0, p, p, 0, z, z, p, table, lens, ctypes.byref(sh),
                                                             0, 1, 0.9, 0.9, act, z)
    assert fwd(z, p, p) == -1
    assert fwd(p, odd4, z) == -7
    assert fwd(p, z, odd4) == -7
    assert fwd(p, p, p, act=9) == -4
    assert h.ncn_inverse_indexed(p, p, 0, z, p, 0, p, p, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -1
    assert h.ncn_inverse_indexed(p, p, 0, p, p, 0, p, odd4, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -7
    args = [p, p, 0, p, p, 0, p, p, 0, z, z, p, p]
    ws = h.ncn_workspace_bytes(ctypes.byref(sh))
    assert h.ncn_backward_indexed(*args, p, ctypes.c_size_t(ws - 1), p, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -5
    assert h.ncn_backward_indexed(*args, p, ctypes.c_size_t(ws), odd4, p, ctypes.byref(sh), 0, 1, 0.9, 0.9, 0, z) == -7
    bad = _shape(lib, 2, 66, 32, 4, 4)
    assert h.ncn_backward_indexed(*args, p, ctypes.c_size_t(ws), p, p, ctypes.byref(bad), 0, 1, 0.9, 0.9, 0, z) == -2


def test_radix_plan_and_argument_checks(lib):
    h = lib.load()
    buf = (ctypes.c_int32 * 96)()
    deep = _shape(lib, 128, 8192, 128, 4, 2)
    assert h.ncn_plan_radix(ctypes.byref(deep), 0, 13, 0, 0, buf, 16) == 2
    assert list(buf[0:6]) == [0, 8, 1, 1, 256, 256] and list(buf[6:12]) == [8, 5, 1, 256, 32, 256]
    assert h.ncn_plan_radix(ctypes.byref(deep), 0, 13, 0, 1, buf, 16) == 2
    assert list(buf[0:6]) == [0, 7, 1, 1, 128, 128] and list(buf[6:12]) == [7, 6, 1, 128, 64, 128]
    assert h.ncn_plan_radix(ctypes.byref(deep), 0, 14, 0, 0, None, 0) == -2          # 2^14 > N
    assert h.ncn_plan_radix(ctypes.byref(_shape(lib, 2, 96, 32, 2, 2)), 0, 6, 0, 0, None, 0) == -2   # 64 does not divide 96
    assert h.ncn_plan_radix(ctypes.byref(_shape(lib, 2, 96, 32, 2, 2)), 0, 5, 0, 0, buf, 16) == 1
    assert list(buf[0:6]) == [0, 5, 1, 1, 32, 96]                                    # three windows per workgroup
    # every plan covers every row: N = odd * n^k leaves a window count that the per-workgroup count must divide
    for n, ec in ((2, 32), (4, 32), (2, 16), (4, 16), (8, 32)):
        for N in [n ** k * odd for k in range(1, 9) for odd in (1, 3, 5, 7, 9, 15) if n ** k * odd <= 4096]:
            kmax = 0
            while N % n ** (kmax + 1) == 0:
                kmax += 1
            for first in range(kmax):
                for count in range(1, kmax - first + 1):
                    for backward in (0, 1):
                        sh = _shape(lib, 1, N, 4 * ec, 4, n)
                        k = h.ncn_plan_radix(ctypes.byref(sh), first, count, 0, backward, buf, 16)
                        assert 0 < k <= 16, (n, N, first, count, backward, k)
                        nxt = 0
                        for q in range(k):
                            f, c, multi, s0, span, rows = buf[6 * q:6 * q + 6]
                            assert f == nxt and c >= 1 and s0 == n ** (first + f) and span == n ** c
                            nxt = f + c
                            if multi:   # a whole number of windows per workgroup, a whole number of workgroups per entry
                                assert rows % span == 0 and N % rows == 0, (n, N, first, count, backward, q, rows)
                                assert rows * ec * 4 * (4 if backward else 2) <= 64 * 1024
                        assert nxt == count
    small = _shape(lib, 2, 64, 32, 4, 4)
    p = ctypes.c_void_p(4096)       # never dereferenced: every call below fails validation first
    z = ctypes.c_void_p(0)
    fwd = lambda x, first, count: h.ncn_forward_radix(x, p, 0, p, p, 0, z, z, p, ctypes.byref(small), first, count,
                                                      0.9, 0.9, 0, z)
    assert fwd(z, 0, 3) == -1
    assert fwd(p, 0, 4) == -2 and fwd(p, 2, 2) == -2 and fwd(p, -1, 1) == -2
    args = [p, p, 0, p, p, 0, p, p, 0, z, z, p, p]
    ws = h.ncn_workspace_bytes(ctypes.byref(small))
    bwd = lambda nbytes, count, dxt=0: h.ncn_backward_radix(*args[:8], dxt, *args[9:], p, ctypes.c_size_t(nbytes),
                                                            ctypes.byref(small), 0, count, 0.9, 0.9, 0, z)
    assert bwd(ws - 1, 1) == -5
    assert bwd(ws, 3) == -8             # several levels carry their state in x_rec, xa_rec


def test_python_grouping_validation():
    from ncn_cuda_amd import ncn_cuda_module as M
    good = torch.randperm(64)
    M.validate_grouping(good, torch.tensor([3, 64]), batch=2, N=64, n_stages=1)
    M.validate_grouping(None, None, batch=2, N=64, n_stages=1)
    M.check_group_table(good, 64)
    M.check_group_table(torch.stack([good, good.flip(0)]), 64)
    with pytest.raises(ValueError, match="permutation"):
        M.check_group_table(torch.zeros(64, dtype=torch.int64), 64)
    with pytest.raises(ValueError, match="group_index"):
        M.validate_grouping(good[:-1], None, batch=2, N=64, n_stages=1)
    with pytest.raises(ValueError, match="group_index"):
        M.validate_grouping(good, None, batch=2, N=64, n_stages=2)
    with pytest.raises(ValueError, match="ctx_len"):
        M.validate_grouping(None, torch.tensor([1, 2, 3]), batch=2, N=64, n_stages=1)
    with pytest.raises(TypeError):
        M.validate_grouping(good.float(), None, batch=2, N=64, n_stages=1)
    with pytest.raises(TypeError):
        M.validate_grouping([1, 2, 3], None, batch=2, N=64, n_stages=1)
    x = torch.zeros(2, 64, 32)
    with pytest.raises(RuntimeError, match="GPU"):      # tables do not open a CPU path either
        M.forward_stages(x, x, torch.zeros(64), 0.9, 0, 4, 4, 0, 1, group_index=good)


def test_python_validation_mirrors_reference_asserts():
    from ncn_cuda_amd import ncn_cuda_module as M
    x = torch.randn(2, 32, 16)
    W = torch.randn(32)
    with pytest.raises(ValueError, match="block_size must divide N"):   # torch_ref/ncn_pytorch.py:25
        M.forward(x, x, W, 0.9, 0, 5, 2, 0)
    with pytest.raises(ValueError, match="n_head must divide E"):
        M.forward(x, x, W, 0.9, 0, 4, 3, 0)
    with pytest.raises(ValueError, match="2E"):
        M.forward(x, x, W[:-1], 0.9, 0, 4, 2, 0)
    with pytest.raises(ValueError, match="activation"):
        M.forward(x, x, W, 0.9, 9, 4, 2, 0)
    with pytest.raises(ValueError, match="same shape"):
        M.forward(x, x[:, :16], W, 0.9, 0, 4, 2, 0)
    with pytest.raises(TypeError):
        M.forward(x.double(), x.double(), W, 0.9, 0, 4, 2, 0)
    with pytest.raises(ValueError, match="unsupported"):
        M.forward(torch.randn(1, 256, 16), torch.randn(1, 256, 16), W, 0.9, 0, 128, 2, 0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):           # product path never runs on the CPU
        M.forward(x, x, W, 0.9, 0, 4, 2, 0)


def test_surface_matches_reference_names():
    import inspect

    import ncn_cuda_amd as pkg
    def positional(fn):  # keyword-only extras (fuse_stages, save_every) are additions, not part of the reference
        return [n for n, q in inspect.signature(fn).parameters.items() if q.kind != q.KEYWORD_ONLY]

    assert list(inspect.signature(pkg.fused_ncn_cuda_v2).parameters) == [
        "x", "xa", "W", "alpha", "activation", "n_cache", "n_head", "module_l"]
    assert positional(pkg.NCNModuleCuda.__init__)[1:] == [
        "alpha", "activation", "n_cache", "n_head", "module_nr", "embed_dim"]
    assert positional(pkg.NCNNetCuda.__init__)[1:] == [
        "alpha", "activation", "n_cache", "n_head", "num_modules", "embed_dim"]
    assert positional(pkg.NCNNetTestCuda.__init__)[1:] == [
        "alpha", "activation", "n_cache", "n_head", "num_modules", "weights"]
    net = pkg.NCNNetCuda(0.9, "tanh", 4, 2, 3, 16)
    assert sorted(net.state_dict()) == ["ncn_modules.0.weight", "ncn_modules.1.weight", "ncn_modules.2.weight"]
    assert net.ncn_modules[1].weight.shape == (32,)
    reference_map = {"tanh": 0, "relu": 1, "sigmoid": 2, "linear": -1}  # ncn_pytorch_wrapper_v2.py:111
    assert {k: pkg.ACTIVATION_CODES[k] for k in reference_map} == reference_map
    assert pkg.ACTIVATION_CODES["leaky-relu"] == 3 and len(pkg.ACTIVATION_CODES) == 5


def test_triton_surface_names_and_arguments():
    """ncn_triton/ncn_triton.py:333-421 by name and positional arguments; activation names map to codes."""
    import inspect
    from ncn_cuda_amd import ncn_triton as T
    assert list(inspect.signature(T.fused_ncn_triton).parameters) == [
        "x", "xa", "W", "ALPHA", "ACTIVATION", "NHEAD", "CACHE", "MODULE_L"]
    ctor = ["alpha", "activation", "n_cache", "n_head"]
    assert list(inspect.signature(T.NCNModuleTriton.__init__).parameters)[1:] == ctor + ["module_nr", "embed_dim"]
    assert list(inspect.signature(T.NCNNetTriton.__init__).parameters)[1:] == ctor + ["num_modules", "embed_dim"]
    assert list(inspect.signature(T.NCNNetTestTriton.__init__).parameters)[1:] == ctor + ["num_modules", "weights"]
    assert [T.activation_code(a) for a in ("tanh", "leaky-relu", "none", "relu", 2)] == [0, 3, -1, -1, 2]
    net = T.NCNNetTriton(0.9, "tanh", 4, 2, 3, 16)
    assert sorted(net.state_dict()) == [f"ncn_modules.{l}.weight" for l in range(3)]
    assert net.ncn_modules[0].weight.shape == (32,) and net.ncn_modules[0].weight.std() < 0.1
    net.ncn_modules[1].reset_parameters()
    assert net.ncn_modules[1].weight.abs().max() <= 0.25


def test_product_code_never_imports_the_oracle():
    pkg_dir = os.path.join(ROOT, "ncn_cuda_amd")
    for dirpath, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".h", ".hip")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "never", (dirpath, f)


def _passes(lib, shape, first, count, backward):
    buf = (ctypes.c_int32 * (8 * 32))()
    k = lib.load().ncn_plan_passes(ctypes.byref(shape), first, count, 0, int(backward), buf, 32)
    assert 0 <= k <= 32
    return [tuple(buf[8 * j:8 * j + 8]) for j in range(k)]


def test_planner_puts_stages_where_they_cost_least(lib):
    """The 13 stages of the deep configuration.  Backward: the pass that runs last (stages 0-2) writes gradients only
    and is bound by instruction issue, the middle pass by its traffic, where a third stage is free: stages 3-5 go
    there, not a fourth stage into the last pass (both cuts move the same bytes).  Forward: two passes."""
    shape = _shape(lib, 128, 8192, 128, 4, 2)
    bwd = _passes(lib, shape, 0, 13, True)
    assert [(p[0], p[1], p[2]) for p in bwd] == [(0, 3, 1), (3, 3, 1), (6, 7, 2)]      # (first, count, 1 halo / 2 closed)
    assert [(p[4], p[6]) for p in bwd] == [(128, 122), (128, 114), (128, 128)]         # (window, owned groups)
    fwd = _passes(lib, shape, 0, 13, False)
    assert [(p[0], p[1], p[2]) for p in fwd] == [(0, 5, 1), (5, 8, 2)]


def test_one_feature_heads_are_planned_as_heads_of_adjacent_ones(lib):
    """E == n_head: the passes, and the workspace that goes with them, are those of E / w heads of w features, w the
    largest of 32, 16, 8, 4 that divides E; at w = 4 there are no multi-stage passes."""
    h = lib.load()
    for E, w in ((128, 32), (48, 16), (24, 8)):
        one, wide = _shape(lib, 4, 8192, E, E, 2), _shape(lib, 4, 8192, E, E // w, 2)
        for backward in (False, True):
            assert _passes(lib, one, 0, 13, backward) == _passes(lib, wide, 0, 13, backward) != []
        for b in (0, 1, 2):
            assert (h.ncn_workspace_bytes_stages(ctypes.byref(one), 0, 13, 0, b)
                    == h.ncn_workspace_bytes_stages(ctypes.byref(wide), 0, 13, 0, b))
    assert _passes(lib, _shape(lib, 4, 8192, 12, 12, 2), 0, 13, True) == []     # four heads to a row: one launch per stage
    assert _passes(lib, _shape(lib, 4, 8192, 6, 6, 2), 0, 13, True) == []       # generic kernels


@pytest.mark.parametrize("backward", [False, True])
@pytest.mark.parametrize("dims", [(128, 8192, 128, 4, 2, 0, 13), (32, 1024, 128, 4, 4, 0, 5), (3, 1024, 64, 2, 2, 0, 11),
                                  (2, 2048, 64, 2, 2, 3, 6), (5, 64, 128, 4, 4, 0, 3), (1, 1 << 16, 32, 1, 2, 0, 20),
                                  (3, 2048, 16, 2, 2, 0, 10), (2, 2048, 128, 2, 2, 0, 11), (2, 1024, 32, 4, 4, 0, 6),
                                  (2, 512, 128, 2, 4, 0, 6),                      # heads of 8 and of 64 features
                                  (2, 2048, 256, 2, 2, 0, 11), (2, 1024, 128, 1, 4, 5, 4),   # heads of 128 features
                                  (2, 3 * 512, 64, 2, 2, 0, 12), (2, 96, 32, 4, 4, 0, 6), (2, 3 * 4096, 128, 4, 2, 0, 14),
                                  (2, 5 * 256, 64, 2, 2, 0, 9), (2, 7 * 64, 32, 2, 4, 2, 5)])  # 3, 5, 7 times a power of two
def test_multi_stage_plan_invariants(lib, dims, backward):
    """The pass planner (host logic): passes tile the stage range in order; a halo window owns what its halo leaves,
    and the halo is (n_cache - 1) * sum of the pass's strides in sub-blocks; closed passes own their whole window."""
    batch, N, E, C, n, first, count = dims
    shape = _shape(lib, batch, N, E, C, n)
    groups = N // n
    passes = _passes(lib, shape, first, count, backward)
    assert passes, "these shapes are eligible for multi-stage passes"
    nxt = 0
    for (p_first, p_count, kind, s0, window, halo, own, cgroups) in passes:
        assert p_first == nxt and p_count >= 1
        nxt += p_count
        strides = [(0 if (first + p_first + k) == 0 else pow(2, first + p_first + k - 1, groups)) for k in range(p_count)]
        if kind == 0:
            assert p_count == 1
            continue
        assert p_count >= 2 and p_count <= 8
        assert window <= groups
        nz = [s for s in strides if s]
        assert s0 & (s0 - 1) == 0 and groups % s0 == 0 and all(s % s0 == 0 for s in nz)   # classes: residues modulo S0
        ring = groups // s0
        # rows a workgroup keeps in LDS: groups of two rows leave their slot-0 rows in registers
        lds_bytes = window * (1 if n == 2 else n) * (E // C) * 4 * (4 if backward else 2)
        assert lds_bytes <= 64 * 1024
        if kind == 2:
            assert window % ring == 0 and halo == 0 and own == window and cgroups * (window // ring) == s0
            rings = window // ring
            assert rings & (rings - 1) == 0                       # whole rings, a power of two of them
        else:
            assert ring > window and cgroups == s0 and window & (window - 1) == 0
            assert halo == (n - 1) * sum(s // s0 for s in strides)
            assert own == window - 2 * halo and 4 * own >= 3 * window
    assert nxt == count


def test_multi_stage_plan_declines_ineligible_shapes(lib):
    assert _passes(lib, _shape(lib, 128, 4096, 128, 4, 16), 0, 3, False) == []   # n_cache = 16: arithmetic-bound
    assert _passes(lib, _shape(lib, 2, 60, 32, 4, 4), 0, 3, False) == []         # 15 groups: no power of two divides them
    assert _passes(lib, _shape(lib, 2, 96, 32, 4, 4), 0, 3, False) != []         # 24 groups = 3 * 8: classes modulo 2, 4, 8
    assert _passes(lib, _shape(lib, 2, 1024, 128, 4, 2), 0, 1, False) == []      # a single stage
    # the deep configuration: three passes forward, four at most backward, closed rings last
    fwd = _passes(lib, _shape(lib, 128, 8192, 128, 4, 2), 0, 13, False)
    assert [p[2] for p in fwd][-1] == 2 and len(fwd) <= 4


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No fallback: if libncn_hip.so is absent and cannot be built, the binding raises instead of computing something
    else."""
    from ncn_cuda_amd import _build, _lib

    def no_compiler():
        raise RuntimeError("hipcc not found")

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libncn_hip.so"))
    monkeypatch.setattr(_build, "build", no_compiler)
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_header_is_valid_c(tmp_path):
    """include/ncn_hip.h is a C header: a C translation unit that only includes it and takes the address of every
    entry point must compile with gcc -std=c99 -Wall -Werror."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    names = _declared_functions()
    body = "\n".join(f"    p[{k}] = (void*)&{n};" for k, n in enumerate(names))
    src.write_text(f'#include "ncn_hip.h"\nvoid* p[{len(names)}];\nvoid take(void) {{\n{body}\n}}\n'
                   "int size_ok[sizeof(ncn_shape) == 32 ? 1 : -1];\n")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-Wno-pedantic", "-I", os.path.join(ROOT, "include"), "-c",
                    str(src), "-o", str(tmp_path / "use_header.o")], check=True)


def test_library_staleness_check(lib, monkeypatch, tmp_path):
    """load() builds a library that is missing or was made from other sources instead of failing: the check behind it
    compares contents (the build id compiled into the library against a hash of the sources), never file times."""
    import shutil
    from ncn_cuda_amd import _build
    assert lib._stale_reason() is None                      # what build() left carries the hash of these sources
    assert lib.load().ncn_build_id().decode() == _build.source_build_id() == _build.library_build_id()
    # a source whose time stamp is newer than the library, content unchanged: not stale, and nothing to compile
    src = os.path.join(_build.CSRC, "ncn_device.h")
    before = os.stat(src)
    try:
        os.utime(src, None)
        assert os.path.getmtime(src) > os.path.getmtime(_build.LIB_PATH)
        assert lib._stale_reason() is None
        assert _build.build(force=False) == []
    finally:
        os.utime(src, (before.st_atime, before.st_mtime))
    # a library older than everything (as after a copy that keeps no times) is still current
    lib_before = os.stat(_build.LIB_PATH)
    try:
        os.utime(_build.LIB_PATH, (1, 1))
        assert lib._stale_reason() is None
    finally:
        os.utime(_build.LIB_PATH, (lib_before.st_atime, lib_before.st_mtime))
    # changed content is what makes it stale: the same sources with one byte more in a header
    copy = tmp_path / "csrc"
    shutil.copytree(_build.CSRC, copy)
    with open(copy / "ncn_device.h", "a") as fh:
        fh.write("\n")
    monkeypatch.setattr(_build, "CSRC", str(copy))
    assert _build.source_build_id() != _build.library_build_id()
    assert "other sources" in lib._stale_reason()
    monkeypatch.undo()
    # no library at all
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "libncn_hip.so"))
    assert "missing" in lib._stale_reason()


def test_stale_library_without_compiler_loads_with_a_warning(lib, monkeypatch, capsys):
    """A box without hipcc and a library that does not match its sources: load it and say so, rather than fail."""
    from ncn_cuda_amd import _build
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "_stale_reason", lambda: "libncn_hip.so was built from other sources (test)")
    monkeypatch.setattr(_build, "have_hipcc", lambda: False)
    monkeypatch.setattr(_build, "build", lambda **kw: (_ for _ in ()).throw(AssertionError("must not build")))
    assert lib.load() is not None
    assert "no hipcc here" in capsys.readouterr().err


def test_python_validation_rejects_scalars_no_kernel_takes(lib):
    """alpha next to zero runs on the generic kernels, which take heads of up to 64 features: a clear error beyond."""
    from ncn_cuda_amd import ncn_cuda_module as M
    x = torch.zeros(1, 16, 256)
    W = torch.zeros(512)
    M.validate(x, x, W, 4, 2, 0, alpha=0.9, m=0.9)            # heads of 128: register kernels
    M.validate(torch.zeros(1, 16, 64), torch.zeros(1, 16, 64), torch.zeros(128), 4, 2, 0, alpha=1e-5)   # generic
    with pytest.raises(ValueError, match="generic kernels"):
        M.validate(x, x, W, 4, 2, 0, alpha=1e-5, m=0.9)


def test_probe_entry_points_validate_their_arguments(lib):
    """The measurement aid: modes are described without a GPU, bad arguments are refused before any launch."""
    h = lib.load()
    valu, flops = ctypes.c_int(0), ctypes.c_int(0)
    assert h.ncn_probe_issue_info(0, ctypes.byref(valu), ctypes.byref(flops)) == 8 and (valu.value, flops.value) == (1, 2)
    assert h.ncn_probe_issue_info(8, ctypes.byref(valu), ctypes.byref(flops)) == 8 and (valu.value, flops.value) == (20, 28)
    assert h.ncn_probe_issue_info(15, ctypes.byref(valu), ctypes.byref(flops)) == 8 and (valu.value, flops.value) == (1, 0)
    assert h.ncn_probe_issue_info(16, None, None) == -2
    assert h.ncn_probe_issue_info(99, None, None) == -2
    p = ctypes.c_void_p(4096)
    assert h.ncn_probe_issue(0, 8, 8, 16, None, None) == -1
    assert h.ncn_probe_issue(99, 8, 8, 16, p, None) == -2
    assert h.ncn_probe_issue(0, 3, 8, 16, p, None) == -2      # chains: 1, 4 or 8
    assert h.ncn_probe_issue(0, 8, 3, 16, p, None) == -2      # waves per SIMD: 1, 2, 4 or 8
