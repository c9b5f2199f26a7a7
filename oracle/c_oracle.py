"""ctypes binding and build recipe of oracle/ncn_oracle.c -- TEST INFRASTRUCTURE ONLY (see that file's header).

build() compiles the C restatement twice (float and double) into oracle/libncn_oracle.so with gcc; the CPU tests, and
the cpu_baseline leg of bench.py, load it.  The shipped package never does.
"""
import ctypes
import os
import shutil
import subprocess

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libncn_oracle.so")
SRC = os.path.join(HERE, "ncn_oracle.c")
# No -march=native: the library is built in one container and run on another machine.  No -ffast-math either: this is
# a checker.
CFLAGS = ["-O3", "-fPIC", "-fopenmp", "-std=c11", "-fno-math-errno"]


def build(verbose=False):
    gcc = shutil.which("gcc")
    if not gcc:
        raise RuntimeError("gcc not found: cannot build oracle/libncn_oracle.so")
    objs = []
    for real, suffix in (("float", "_f32"), ("double", "_f64")):
        obj = os.path.join(HERE, f"ncn_oracle{suffix}.o")
        cmd = [gcc, *CFLAGS, f"-DREAL={real}", f"-DSUFFIX={suffix}", "-c", SRC, "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"gcc failed:\n{proc.stdout}\n{proc.stderr}")
        objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    proc = subprocess.run([gcc, "-shared", "-fopenmp", "-o", tmp, *objs, "-lm"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    for obj in objs:
        os.remove(obj)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


_lib = None


def load():
    """The built library (built on first use if it is not there: gcc takes a second)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        vp, i64, i = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        for suffix, real in (("_f32", ctypes.c_float), ("_f64", ctypes.c_double)):
            f = getattr(lib, "ncn_ref_stage_forward" + suffix)
            f.restype = i
            f.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i, i, i64, real, real, i, i, vp, vp]
            b = getattr(lib, "ncn_ref_stage_backward" + suffix)
            b.restype = i
            b.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i, i, i64, real, real, i, vp, vp]
            getattr(lib, "ncn_ref_threads" + suffix).restype = i
        _lib = lib
    return _lib


def threads():
    return load().ncn_ref_threads_f32()


def _suffix(t):
    if t.dtype == torch.float32:
        return "_f32"
    if t.dtype == torch.float64:
        return "_f64"
    raise TypeError("the C oracle takes float32 or float64 CPU tensors")


def _c(t):
    if t.device.type != "cpu":
        raise ValueError("the C oracle takes CPU tensors")
    return t.contiguous()


def _i32(t, count, what):
    """An optional int32 array for the C side (None stays NULL); the caller keeps the returned tensor alive."""
    if t is None:
        return None, None
    t = torch.as_tensor(t).to(torch.int32).contiguous()
    if t.numel() != count:
        raise ValueError(f"{what} must have {count} entries")
    return t, t.data_ptr()


def stage_forward(X, Xa, W, alpha, n, C, stage, m=0.9, activation=0, inverse=False, table=None, ctx_len=None):
    """One stage (or its inverse) on CPU tensors [batch, N, E]; returns (Y, Ya).  `table` [N] replaces the stride
    map (position of slot o of group g at entry g*n + o), `ctx_len` [batch] gives each batch entry its live slots."""
    X, Xa, W = _c(X), _c(Xa), _c(W).to(X.dtype)
    Y, Ya = torch.empty_like(X), torch.empty_like(Xa)
    batch, N, E = X.shape
    tk, tp = _i32(table, N, "table")
    lk, lp = _i32(ctx_len, batch, "ctx_len")
    rc = getattr(load(), "ncn_ref_stage_forward" + _suffix(X))(
        X.data_ptr(), Xa.data_ptr(), Y.data_ptr(), Ya.data_ptr(), W.data_ptr(), batch, N, E, C, n, stage, alpha, m,
        activation, 1 if inverse else 0, tp, lp)
    if rc:
        raise ValueError(f"C oracle refused the shape (rc {rc})")
    return Y, Ya


def net_forward(x, xa, weights, alpha, n, C, m=0.9, activation=0, first_stage=0):
    for l, W in enumerate(weights):
        x, xa = stage_forward(x, xa, W, alpha, n, C, first_stage + l, m, activation)
    return x, xa


def net_inverse(y, ya, weights, alpha, n, C, m=0.9, activation=0, first_stage=0):
    for l in range(len(weights) - 1, -1, -1):
        y, ya = stage_forward(y, ya, weights[l], alpha, n, C, first_stage + l, m, activation, inverse=True)
    return y, ya


def stage_backward(Y, Ya, dY, dYa, W, alpha, n, C, stage, m=0.9, activation=0, table=None, ctx_len=None):
    """Reversible backward of one stage from its outputs; returns (x_rec, xa_rec, dx, dxa, dW[2E] float64)."""
    Y, Ya, dY, W = _c(Y), _c(Ya), _c(dY), _c(W).to(Y.dtype)
    dYa = _c(dYa) if dYa is not None else None
    xr, xar, dx, dxa = (torch.empty_like(Y) for _ in range(4))
    batch, N, E = Y.shape
    dW = torch.empty(2 * E, dtype=torch.float64)
    tk, tp = _i32(table, N, "table")
    lk, lp = _i32(ctx_len, batch, "ctx_len")
    rc = getattr(load(), "ncn_ref_stage_backward" + _suffix(Y))(
        Y.data_ptr(), Ya.data_ptr(), dY.data_ptr(), dYa.data_ptr() if dYa is not None else None, W.data_ptr(),
        xr.data_ptr(), xar.data_ptr(), dx.data_ptr(), dxa.data_ptr(), dW.data_ptr(), batch, N, E, C, n, stage, alpha, m,
        activation, tp, lp)
    if rc:
        raise ValueError(f"C oracle refused the shape (rc {rc})")
    return xr, xar, dx, dxa, dW


def net_forward_backward(x, xa, weights, dy, dya, alpha, n, C, m=0.9, activation=0, first_stage=0, tables=None,
                         ctx_len=None, keep_outputs=True):
    """Forward keeping every stage's outputs, then the reversible backward stage by stage (what an autograd node per
    stage does).  keep_outputs=False keeps only the last stage's outputs and lets each backward stage hand the
    inputs it reconstructs to the one below (for float64 runs on tensors too large to keep L copies of).  `tables`
    is a list of one table per stage.  Returns (yi, ya, dx, dxa, [dW_l])."""
    outs = []
    tab = lambda l: None if tables is None else tables[l]
    for l, W in enumerate(weights):
        x, xa = stage_forward(x, xa, W, alpha, n, C, first_stage + l, m, activation, table=tab(l), ctx_len=ctx_len)
        if keep_outputs:
            outs.append((x, xa))
    yi, ya = x, xa
    g, h = dy, dya
    dWs = [None] * len(weights)
    for l in range(len(weights) - 1, -1, -1):
        cy, cya = outs.pop() if keep_outputs else (x, xa)
        x, xa, g, h, dWs[l] = stage_backward(cy, cya, g, h, weights[l], alpha, n, C, first_stage + l, m, activation,
                                             table=tab(l), ctx_len=ctx_len)
    return yi, ya, g, h, dWs


if __name__ == "__main__":
    build(verbose=True)
