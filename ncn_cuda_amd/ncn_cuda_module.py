"""Tensor-level entry points with the signatures of the reference's pybind11 module.

The reference builds `ncn_cuda_module` from ncn_cuda/ncn_cuda.cpp:29-32 and exposes

    forward(X, Xa, W, alpha, activation, cache_dim, nhead, module_l)            -> [Y, Ya]
    backward(Y, Ya, dY, dYa, W, alpha, activation, cache_dim, nhead, module_l)  -> [X, Xa, dX, dXa, dW]

This module offers the same two callables (plus `inverse` and the multi-stage variants) on top of
libncn_hip.so.  Tensors are allocated here with torch.empty; the library itself never allocates.
Deviations from the reference module, all visible in the signatures or return values:
  * `dW` comes back already summed over batch and positions, shaped [1, 1, 2E], so that the
    reference wrapper's `torch.sum(dW, dim=(0, 1))` (ncn_pytorch_wrapper_v2.py:48) still yields
    the [2E] gradient (the reference returns per-row partials [batch, N, 2E]);
  * float32 and bfloat16 activations are accepted (reference: float32 only); W may be either and is
    used as float32;
  * launches go to the current PyTorch stream and do not synchronise the host;
  * invalid arguments raise ValueError/TypeError instead of reading out of bounds.
"""
import ctypes
import weakref

import torch

from . import _lib

M_DEFAULT = 0.9  # hard-coded by the reference: ncn_fwd_cuda_kernel.cu:72, ncn_pytorch.py:89

_DTYPES = {torch.float32: _lib.NCN_F32, torch.bfloat16: _lib.NCN_BF16}
_ACT_CODES = (_lib.ACT_TANH, _lib.ACT_RELU, _lib.ACT_SIGMOID, _lib.ACT_LEAKY_RELU, _lib.ACT_LINEAR)


def validate(x, xa, W, n_cache, n_head, activation, module_l=0, n_stages=1, what="x", alpha=None, m=None):
    """Host-side argument checks (no GPU needed).  Raises TypeError / ValueError.  With alpha (and m) also checks that
    some kernel takes these scalars at this head width."""
    if not (isinstance(x, torch.Tensor) and isinstance(xa, torch.Tensor) and isinstance(W, torch.Tensor)):
        raise TypeError("x, xa and W must be torch tensors")
    if x.dim() != 3:
        raise ValueError(f"{what} must be [batch, N, E], got shape {tuple(x.shape)}")
    if xa.shape != x.shape:
        raise ValueError(f"{what} and its companion must have the same shape, got {tuple(x.shape)} and {tuple(xa.shape)}")
    if x.dtype not in _DTYPES or xa.dtype != x.dtype:
        raise TypeError(f"activations must both be float32 or bfloat16, got {x.dtype} and {xa.dtype}")
    if W.dtype not in _DTYPES:
        raise TypeError(f"W must be float32 or bfloat16, got {W.dtype}")
    batch, N, E = x.shape
    n_cache, n_head, module_l, n_stages = int(n_cache), int(n_head), int(module_l), int(n_stages)
    if batch <= 0 or N <= 0 or E <= 0:
        raise ValueError(f"empty tensor of shape {tuple(x.shape)}")
    if n_cache <= 0 or N % n_cache != 0:
        raise ValueError(f"block_size must divide N (N={N}, n_cache={n_cache})")
    if n_head <= 0 or E % n_head != 0:
        raise ValueError(f"n_head must divide E (E={E}, n_head={n_head})")
    if module_l < 0 or n_stages < 1:
        raise ValueError(f"bad stage range: first stage {module_l}, {n_stages} stages")
    if W.numel() != n_stages * 2 * E:
        raise ValueError(f"W must hold {n_stages} x 2E = {n_stages * 2 * E} values, got {W.numel()}")
    if int(activation) not in _ACT_CODES:
        raise ValueError(f"unknown activation code {activation} (0 tanh, 1 relu, 2 sigmoid, 3 leaky relu, -1 linear)")
    shape = _lib.NcnShape(batch, N, E, n_head, n_cache)
    rc = _lib.load().ncn_check_shape(ctypes.byref(shape), module_l, n_stages, int(activation))
    if rc != 0:
        raise ValueError(f"unsupported NCN problem {tuple(x.shape)}, n_cache={n_cache}, n_head={n_head}: "
                         f"{_lib.error_string(rc)}")
    if alpha is not None:
        mm = M_DEFAULT if m is None else float(m)
        if _lib.load().ncn_kernel_path_scalars(ctypes.byref(shape), float(alpha), mm) == 0:
            raise ValueError(f"alpha={alpha}, m={mm} with heads of {E // n_head} features: the register kernels take "
                             "alpha in [1e-3, 1e3] and m in [1e-3, 0.999], and the generic kernels, which take any "
                             "scalars, only heads of up to 64 features")
    return shape


def _require_gpu(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("the NCN kernels run on the GPU only: got a CPU tensor (there is no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"all tensors must live on one device, got {dev} and {t.device}")
    return dev


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _prep(t):
    """Contiguous, 16-byte aligned view or copy."""
    t = t.contiguous()
    if t.data_ptr() % 16 != 0:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _w32(W):
    return _prep(W.detach().reshape(-1).to(torch.float32))


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def validate_grouping(group_index, ctx_len, batch, N, n_stages):
    """Host-side checks of a grouping table [n_stages, N] (or [N] for one stage) and of context lengths [batch];
    either may be None.  Shapes and dtypes only: whether the table is a permutation is checked by
    check_group_table, which needs the values."""
    for name, t in (("group_index", group_index), ("ctx_len", ctx_len)):
        if t is None:
            continue
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch tensor")
        if t.dtype not in (torch.int32, torch.int64):
            raise TypeError(f"{name} must be int32 or int64, got {t.dtype}")
    if group_index is not None and group_index.numel() != n_stages * N:
        raise ValueError(f"group_index must hold {n_stages} x N = {n_stages * N} positions, got {group_index.numel()}")
    if ctx_len is not None and ctx_len.numel() != batch:
        raise ValueError(f"ctx_len must hold one length per batch entry ({batch}), got {ctx_len.numel()}")


_checked_tables = {}   # id(tensor) -> (weak reference, version counter, N) of tables found good; dies with the tensor


def check_group_table(group_index, N):
    """Raises ValueError unless every row of the table is a permutation of 0 .. N-1 (the kernels clamp bad entries
    but cannot repair a table).  Works on CPU or GPU tensors; on the GPU it synchronises, so a table that passed is
    remembered (the tensor object with its version counter) and not sorted again while it stays unchanged."""
    key = id(group_index)
    seen = _checked_tables.get(key)
    if seen is not None and seen[0]() is group_index and seen[1:] == (group_index._version, int(N)):
        return
    t = group_index.reshape(-1, N).to(torch.int64)
    want = torch.arange(N, dtype=torch.int64, device=t.device).expand_as(t)
    if not torch.equal(torch.sort(t, dim=1).values, want):
        raise ValueError("group_index: every stage's row must be a permutation of 0 .. N-1")
    _checked_tables[key] = (weakref.ref(group_index, lambda _, k=key: _checked_tables.pop(k, None)),
                            group_index._version, int(N))


def _grouping(group_index, ctx_len, batch, N, n_stages, dev, check_tables):
    validate_grouping(group_index, ctx_len, batch, N, n_stages)
    gi = cl = None
    if group_index is not None:
        _require_gpu(group_index)
        if check_tables:
            check_group_table(group_index, N)
        gi = group_index.detach().reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    if ctx_len is not None:
        cl = ctx_len.detach().reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    return gi, cl


def _is_two_plane(t):
    """A value kept as two bfloat16 planes, [2, batch, N, E]: what forward_stages(save_residual=True) returns."""
    return isinstance(t, torch.Tensor) and t.dim() == 4 and t.shape[0] == 2 and t.dtype == torch.bfloat16


def residual_save_supported(x, n_cache, n_head, alpha=0.9, m=M_DEFAULT):
    """True when forward_stages(save_residual=True) can run this call: the register kernels only."""
    shape = _lib.NcnShape(x.shape[0], x.shape[1], x.shape[2], int(n_head), int(n_cache))
    return _lib.load().ncn_kernel_path_scalars(ctypes.byref(shape), float(alpha), float(m)) == 2


def _check_out(out, like, dtype):
    """The caller's output tensors go to the library as they are: they must be what it will write."""
    if not (isinstance(out, (tuple, list)) and len(out) == 2):
        raise TypeError("out must be a pair of tensors (y, ya)")
    for t in out:
        if not isinstance(t, torch.Tensor):
            raise TypeError("out must hold torch tensors")
        if t.shape != like.shape or t.dtype != dtype or t.device != like.device:
            raise ValueError(f"out tensors must be {tuple(like.shape)} {dtype} on {like.device}, got "
                             f"{tuple(t.shape)} {t.dtype} on {t.device}")
        if not t.is_contiguous() or t.data_ptr() % 16 != 0:
            raise ValueError("out tensors must be contiguous and 16-byte aligned")


def forward_stages(x, xa, W, alpha, activation, cache_dim, nhead, first_stage, n_stages, *, m=M_DEFAULT,
                   out_dtype=None, save_fp32=False, save_residual=False, out=None, group_index=None, ctx_len=None,
                   check_tables=True):
    """Stages first_stage .. first_stage+n_stages-1 in one call.  W: [n_stages, 2E] (any shape with that many
    values).  Returns (y, ya) or, with save_fp32, (y, ya, y32, ya32) where y32/ya32 are float32 copies, or, with
    save_residual (bfloat16 outputs, one stage, register-kernel shapes), (y, ya, ys, yas) where ys, yas are
    [2, batch, N, E] bfloat16: plane 0 is y (the same memory), plane 1 what its rounding took away -- what
    backward_stages takes in place of float32 copies at two thirds of the bytes written.
    group_index [n_stages, N] replaces the stride permutation by a table of positions in (group, slot) order and
    ctx_len [batch] gives every batch entry its own number of live slots (the group_tensor / ctxlen_tensor of
    ncn_triton/ncn_triton_old.py:362-387); rows past the length pass through."""
    shape = validate(x, xa, W, cache_dim, nhead, activation, first_stage, n_stages, alpha=alpha, m=m)
    dev = _require_gpu(x, xa, W)
    indexed = group_index is not None or ctx_len is not None
    gi, cl = _grouping(group_index, ctx_len, x.shape[0], x.shape[1], n_stages, dev, check_tables)
    x, xa, w = _prep(x.detach()), _prep(xa.detach()), _w32(W)
    out_dtype = x.dtype if out_dtype is None else out_dtype
    if out is not None and out_dtype not in _DTYPES:
        raise TypeError(f"out_dtype must be float32 or bfloat16, got {out_dtype}")
    out_code = _DTYPES[out_dtype]
    ys = yas = None
    if save_residual:
        if out_dtype != torch.bfloat16 or n_stages != 1 or save_fp32 or out is not None:
            raise ValueError("save_residual needs bfloat16 outputs, one stage, and neither save_fp32 nor out")
        ys = torch.empty((2,) + tuple(x.shape), dtype=torch.bfloat16, device=dev)
        yas = torch.empty((2,) + tuple(x.shape), dtype=torch.bfloat16, device=dev)
        y, ya = ys[0], yas[0]
        out_code = _lib.NCN_BF16X2
    elif out is not None:
        _check_out(out, x, out_dtype)
        y, ya = out
    else:
        y = torch.empty(x.shape, dtype=out_dtype, device=dev)
        ya = torch.empty(x.shape, dtype=out_dtype, device=dev)
    y32 = ya32 = None
    if save_fp32:
        if out_dtype == torch.float32:
            y32, ya32 = y, ya
        else:
            y32 = torch.empty(x.shape, dtype=torch.float32, device=dev)
            ya32 = torch.empty(x.shape, dtype=torch.float32, device=dev)
    aux = (y32, ya32) if (save_fp32 and out_dtype != torch.float32) else (None, None)
    lib = _lib.load()
    ws, ws_bytes = None, 0
    if indexed:
        with torch.cuda.device(dev):
            rc = lib.ncn_forward_indexed(_ptr(x), _ptr(xa), _DTYPES[x.dtype], _ptr(y), _ptr(ya), out_code,
                                         _ptr(aux[0]), _ptr(aux[1]), _ptr(w), _ptr(gi), _ptr(cl), ctypes.byref(shape),
                                         int(first_stage), int(n_stages), float(alpha), float(m), int(activation),
                                         _stream(dev))
        _lib.check(rc, "ncn_forward_indexed")
        return (y, ya, ys, yas) if save_residual else (y, ya, y32, ya32) if save_fp32 else (y, ya)
    if n_stages > 1:
        ws_bytes = lib.ncn_workspace_bytes_stages(ctypes.byref(shape), int(first_stage), int(n_stages), int(activation), 0)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        rc = lib.ncn_forward(_ptr(x), _ptr(xa), _DTYPES[x.dtype], _ptr(y), _ptr(ya), out_code,
                             _ptr(aux[0]), _ptr(aux[1]), _ptr(w), _ptr(ws), ctypes.c_size_t(ws_bytes),
                             ctypes.byref(shape), int(first_stage), int(n_stages), float(alpha), float(m),
                             int(activation), _stream(dev))
    _lib.check(rc, "ncn_forward")
    return (y, ya, ys, yas) if save_residual else (y, ya, y32, ya32) if save_fp32 else (y, ya)


def forward_stages_saving(x, xa, W, alpha, activation, cache_dim, nhead, stage, *, m=M_DEFAULT, group_index=None,
                          ctx_len=None, check_tables=True):
    """One stage forward, and what an autograd node should keep for backward_stages: returns (y, ya, saved_y, saved_ya).
    float32: the outputs themselves.  bfloat16: the outputs plus what their rounding took away, as two bfloat16 planes
    on the register kernels and as float32 copies on the generic ones (a reversible backward would amplify bare
    bfloat16 rounding by (1/m)^n_cache, 5.4x at 16 rows)."""
    kw = dict(m=m, group_index=group_index, ctx_len=ctx_len, check_tables=check_tables)
    if x.dtype == torch.float32:
        y, ya = forward_stages(x, xa, W, alpha, activation, cache_dim, nhead, stage, 1, **kw)
        return y, ya, y, ya
    if x.dim() == 3 and residual_save_supported(x, cache_dim, nhead, alpha, m):
        return forward_stages(x, xa, W, alpha, activation, cache_dim, nhead, stage, 1, save_residual=True, **kw)
    return forward_stages(x, xa, W, alpha, activation, cache_dim, nhead, stage, 1, save_fp32=True, **kw)


def backward_stages(y, ya, dy, dya, W, alpha, activation, cache_dim, nhead, first_stage, n_stages, *, m=M_DEFAULT,
                    grad_dtype=None, want_inputs=True, group_index=None, ctx_len=None, check_tables=True):
    """Reversible backward of stages first_stage+n_stages-1 .. first_stage from the outputs y, ya of the last one.
    dya may be None (zeros).  y, ya may be the two-plane tensors [2, batch, N, E] of forward_stages(save_residual=True)
    (one stage).  Returns (x_rec, xa_rec, dx, dxa, dW[n_stages, 2E]); x_rec/xa_rec are None when
    want_inputs is False (with several stages the state between them then travels through the workspace and the
    last stage to run writes no reconstructed inputs)."""
    two_plane = _is_two_plane(y) and _is_two_plane(ya)
    if two_plane and n_stages != 1:
        raise ValueError("two-plane saved outputs hold one stage: n_stages must be 1")
    ys_full, yas_full = y, ya
    if two_plane:
        y, ya = ys_full[0], yas_full[0]
    shape = validate(y, ya, W, cache_dim, nhead, activation, first_stage, n_stages, what="y", alpha=alpha, m=m)
    if dy.shape != y.shape or (dya is not None and dya.shape != y.shape):
        raise ValueError("dy/dya must have the shape of y")
    if dy.dtype not in _DTYPES or (dya is not None and dya.dtype != dy.dtype):
        raise TypeError("dy and dya must both be float32 or bfloat16")
    dev = _require_gpu(y, ya, dy, dya, W)
    indexed = group_index is not None or ctx_len is not None
    gi, cl = _grouping(group_index, ctx_len, y.shape[0], y.shape[1], n_stages, dev, check_tables)
    if two_plane:
        y, ya = _prep(ys_full.detach()), _prep(yas_full.detach())
        y_code = _lib.NCN_BF16X2
    else:
        y, ya = _prep(y.detach()), _prep(ya.detach())
        y_code = _DTYPES[y.dtype]
    dy, w = _prep(dy.detach()), _w32(W)
    dya = _prep(dya.detach()) if dya is not None else None
    grad_dtype = dy.dtype if grad_dtype is None else grad_dtype
    need_state = want_inputs
    ws_mode = 1 if want_inputs else 2
    if n_stages > 1 and grad_dtype != torch.float32:
        raise ValueError("multi-stage backward carries its state in float32: use grad_dtype=torch.float32")
    dx = torch.empty(dy.shape, dtype=grad_dtype, device=dev)
    dxa = torch.empty(dy.shape, dtype=grad_dtype, device=dev)
    x_rec = torch.empty(dy.shape, dtype=torch.float32, device=dev) if need_state else None
    xa_rec = torch.empty(dy.shape, dtype=torch.float32, device=dev) if need_state else None
    E = dy.shape[2]
    dW = torch.empty(n_stages, 2 * E, dtype=torch.float32, device=dev)
    lib = _lib.load()
    if indexed:
        # lengths without a table keep the stride permutation: with the multi-stage figure the library runs its
        # multi-stage passes on them too
        if group_index is not None:
            # a table never uses the multi-stage passes: the partial rows of one launch, plus the two float32 arrays
            # (each padded to 256 bytes) that carry the state between stages when no reconstructed inputs are wanted
            plane = (dy.numel() * 4 + 255) // 256 * 256
            ws_bytes = lib.ncn_workspace_bytes(ctypes.byref(shape)) + (2 * plane if ws_mode == 2 and n_stages > 1 else 0)
        else:
            ws_bytes = lib.ncn_workspace_bytes_stages(ctypes.byref(shape), int(first_stage), int(n_stages),
                                                      int(activation), ws_mode)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.ncn_backward_indexed(_ptr(y), _ptr(ya), y_code, _ptr(dy), _ptr(dya), _DTYPES[dy.dtype],
                                          _ptr(dx), _ptr(dxa), _DTYPES[grad_dtype], _ptr(x_rec), _ptr(xa_rec), _ptr(w),
                                          _ptr(dW), _ptr(ws), ctypes.c_size_t(ws_bytes), _ptr(gi), _ptr(cl),
                                          ctypes.byref(shape), int(first_stage), int(n_stages), float(alpha), float(m),
                                          int(activation), _stream(dev))
        _lib.check(rc, "ncn_backward_indexed")
        return x_rec, xa_rec, dx, dxa, dW
    ws_bytes = lib.ncn_workspace_bytes_stages(ctypes.byref(shape), int(first_stage), int(n_stages), int(activation),
                                              ws_mode)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.ncn_backward(_ptr(y), _ptr(ya), y_code, _ptr(dy), _ptr(dya), _DTYPES[dy.dtype],
                              _ptr(dx), _ptr(dxa), _DTYPES[grad_dtype], _ptr(x_rec), _ptr(xa_rec), _ptr(w), _ptr(dW),
                              _ptr(ws), ctypes.c_size_t(ws_bytes), ctypes.byref(shape), int(first_stage),
                              int(n_stages), float(alpha), float(m), int(activation), _stream(dev))
    _lib.check(rc, "ncn_backward")
    return x_rec, xa_rec, dx, dxa, dW


def inverse_stages(y, ya, W, alpha, activation, cache_dim, nhead, first_stage, n_stages, *, m=M_DEFAULT,
                   out_dtype=None, group_index=None, ctx_len=None, check_tables=True, scratch=True):
    """x, xa with forward_stages(x, xa, ...) == (y, ya).  scratch: with several stages, allocate the scratch that lets
    every multi-stage pass run as one (ncn_inverse_ws); without it the stages of a halo pass run one launch each."""
    shape = validate(y, ya, W, cache_dim, nhead, activation, first_stage, n_stages, what="y", alpha=alpha, m=m)
    dev = _require_gpu(y, ya, W)
    indexed = group_index is not None or ctx_len is not None
    gi, cl = _grouping(group_index, ctx_len, y.shape[0], y.shape[1], n_stages, dev, check_tables)
    y, ya, w = _prep(y.detach()), _prep(ya.detach()), _w32(W)
    out_dtype = y.dtype if out_dtype is None else out_dtype
    x = torch.empty(y.shape, dtype=out_dtype, device=dev)
    xa = torch.empty(y.shape, dtype=out_dtype, device=dev)
    if indexed:
        with torch.cuda.device(dev):
            rc = _lib.load().ncn_inverse_indexed(_ptr(y), _ptr(ya), _DTYPES[y.dtype], _ptr(x), _ptr(xa),
                                                 _DTYPES[out_dtype], _ptr(w), _ptr(gi), _ptr(cl), ctypes.byref(shape),
                                                 int(first_stage), int(n_stages), float(alpha), float(m),
                                                 int(activation), _stream(dev))
        _lib.check(rc, "ncn_inverse_indexed")
        return x, xa
    lib = _lib.load()
    ws_bytes = 0
    if scratch and n_stages > 1 and out_dtype == torch.float32:
        ws_bytes = lib.ncn_workspace_bytes_stages(ctypes.byref(shape), int(first_stage), int(n_stages), int(activation), 0)
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.ncn_inverse_ws(_ptr(y), _ptr(ya), _DTYPES[y.dtype], _ptr(x), _ptr(xa), _DTYPES[out_dtype],
                                    _ptr(w), _ptr(ws), ctypes.c_size_t(ws_bytes), ctypes.byref(shape),
                                    int(first_stage), int(n_stages), float(alpha), float(m), int(activation),
                                    _stream(dev))
        _lib.check(rc, "ncn_inverse_ws")
        return x, xa
    with torch.cuda.device(dev):
        rc = lib.ncn_inverse(_ptr(y), _ptr(ya), _DTYPES[y.dtype], _ptr(x), _ptr(xa), _DTYPES[out_dtype],
                             _ptr(w), ctypes.byref(shape), int(first_stage), int(n_stages), float(alpha),
                             float(m), int(activation), _stream(dev))
    _lib.check(rc, "ncn_inverse")
    return x, xa


def forward_radix(x, xa, W, alpha, activation, cache_dim, nhead, first_level, n_levels, *, m=M_DEFAULT,
                  out_dtype=None):
    """Levels first_level .. first_level+n_levels-1 of the radix-n digit grouping (ncn_triton/group_tensors.py:8-18)
    without index tensors; W: [n_levels, 2E].  Several levels per pass stay in LDS for n_cache 2 and 4.  Outputs are
    float32 unless out_dtype says otherwise (values between passes live in the outputs)."""
    shape = validate(x, xa, W, cache_dim, nhead, activation, 0, n_levels, alpha=alpha, m=m)
    dev = _require_gpu(x, xa, W)
    x, xa, w = _prep(x.detach()), _prep(xa.detach()), _w32(W)
    out_dtype = torch.float32 if out_dtype is None else out_dtype
    y = torch.empty(x.shape, dtype=out_dtype, device=dev)
    ya = torch.empty(x.shape, dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().ncn_forward_radix(_ptr(x), _ptr(xa), _DTYPES[x.dtype], _ptr(y), _ptr(ya), _DTYPES[out_dtype],
                                           _ptr(None), _ptr(None), _ptr(w), ctypes.byref(shape), int(first_level),
                                           int(n_levels), float(alpha), float(m), int(activation), _stream(dev))
    if rc == -2:
        raise ValueError(f"radix levels {first_level}..{first_level + n_levels - 1}: n_cache^(last level + 1) must "
                         f"divide N = {x.shape[1]}")
    _lib.check(rc, "ncn_forward_radix")
    return y, ya


def inverse_radix(y, ya, W, alpha, activation, cache_dim, nhead, first_level, n_levels, *, m=M_DEFAULT):
    """x, xa (float32) with forward_radix(x, xa, ...) == (y, ya)."""
    shape = validate(y, ya, W, cache_dim, nhead, activation, 0, n_levels, what="y", alpha=alpha, m=m)
    dev = _require_gpu(y, ya, W)
    y, ya, w = _prep(y.detach()), _prep(ya.detach()), _w32(W)
    x = torch.empty(y.shape, dtype=torch.float32, device=dev)
    xa = torch.empty(y.shape, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().ncn_inverse_radix(_ptr(y), _ptr(ya), _DTYPES[y.dtype], _ptr(x), _ptr(xa), _lib.NCN_F32, _ptr(w),
                                           ctypes.byref(shape), int(first_level), int(n_levels), float(alpha), float(m),
                                           int(activation), _stream(dev))
    if rc == -2:
        raise ValueError(f"radix levels {first_level}..{first_level + n_levels - 1}: n_cache^(last level + 1) must "
                         f"divide N = {y.shape[1]}")
    _lib.check(rc, "ncn_inverse_radix")
    return x, xa


def backward_radix(y, ya, dy, dya, W, alpha, activation, cache_dim, nhead, first_level, n_levels, *, m=M_DEFAULT,
                   want_inputs=True):
    """Reversible backward of forward_radix from its outputs.  Returns (x_rec, xa_rec, dx, dxa, dW[n_levels, 2E]), all
    float32; x_rec, xa_rec are None when want_inputs is False (the library then does not write them)."""
    shape = validate(y, ya, W, cache_dim, nhead, activation, 0, n_levels, what="y", alpha=alpha, m=m)
    if dy.shape != y.shape or (dya is not None and dya.shape != y.shape):
        raise ValueError("dy/dya must have the shape of y")
    if dy.dtype not in _DTYPES or (dya is not None and dya.dtype != dy.dtype):
        raise TypeError("dy and dya must both be float32 or bfloat16")
    dev = _require_gpu(y, ya, dy, dya, W)
    y, ya, dy, w = _prep(y.detach()), _prep(ya.detach()), _prep(dy.detach()), _w32(W)
    dya = _prep(dya.detach()) if dya is not None else None
    f32 = torch.float32
    dx, dxa = torch.empty(y.shape, dtype=f32, device=dev), torch.empty(y.shape, dtype=f32, device=dev)
    x_rec = torch.empty(y.shape, dtype=f32, device=dev) if want_inputs else None
    xa_rec = torch.empty(y.shape, dtype=f32, device=dev) if want_inputs else None
    dW = torch.empty(n_levels, 2 * y.shape[2], dtype=f32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.ncn_workspace_bytes(ctypes.byref(shape))
    if not want_inputs and n_levels > 1:   # two float32 arrays (padded to 256 bytes) carry the state between the passes
        ws_bytes += 2 * ((y.numel() * 4 + 255) // 256 * 256)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.ncn_backward_radix(_ptr(y), _ptr(ya), _DTYPES[y.dtype], _ptr(dy), _ptr(dya), _DTYPES[dy.dtype],
                                    _ptr(dx), _ptr(dxa), _lib.NCN_F32, _ptr(x_rec), _ptr(xa_rec), _ptr(w), _ptr(dW),
                                    _ptr(ws), ctypes.c_size_t(ws_bytes), ctypes.byref(shape), int(first_level),
                                    int(n_levels), float(alpha), float(m), int(activation), _stream(dev))
    if rc == -2:
        raise ValueError(f"radix levels {first_level}..{first_level + n_levels - 1}: n_cache^(last level + 1) must "
                         f"divide N = {y.shape[1]}")
    _lib.check(rc, "ncn_backward_radix")
    return x_rec, xa_rec, dx, dxa, dW


# ---- the reference module's two callables (ncn_cuda/ncn_cuda.cpp:3-25) -------------------------------------
def forward(X, Xa, W, alpha, activation, cache_dim, nhead, module_l):
    y, ya = forward_stages(X, Xa, W, alpha, activation, cache_dim, nhead, module_l, 1)
    return [y, ya]


def backward(Y, Ya, dY, dYa, W, alpha, activation, cache_dim, nhead, module_l):
    x, xa, dx, dxa, dW = backward_stages(Y, Ya, dY, dYa, W, alpha, activation, cache_dim, nhead, module_l, 1)
    return [x, xa, dx, dxa, dW.reshape(1, 1, -1)]


def inverse(Y, Ya, W, alpha, activation, cache_dim, nhead, module_l):
    """Inputs of stage module_l from its outputs (NCNFunctionPytorch.invert,
    torch_ref/ncn_pytorch_invertible.py:87-113, applied for j = cache_dim-1 .. 0)."""
    x, xa = inverse_stages(Y, Ya, W, alpha, activation, cache_dim, nhead, module_l, 1)
    return [x, xa]
