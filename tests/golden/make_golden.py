#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/ from the reference's own CPU definition.

Run once, in the development container only (the reference tree does not exist on the GPU box):

    python tests/golden/make_golden.py [/root/reference]

What it pins.  The layer's arithmetic is fixed by closed forms and invariants, but four
*conventions* are not fixed by any mathematics: how W splits into Wi/Wj per head
(torch_ref/ncn_pytorch.py:60-61), the gather/scatter orientation (:96-97), the step order with the
pre-update x_j shared by all rows (:74-94) and the stage->stride map (:38-40).  The vectors written
here are the only independent guard against transcribing those wrongly, so they are produced by
importing the reference's two pure-PyTorch files and running them on seeded CPU inputs:

  * RefTorchNaive.forward            torch_ref/ncn_pytorch.py:103-124   (+ autograd backward)
  * RefInvTorchNaive.forward         torch_ref/ncn_pytorch_invertible.py:302-358 (+ its custom backward)
  * NCNFunctionPytorch.invert        torch_ref/ncn_pytorch_invertible.py:87-113
  * group_pos_to_index_v2            torch_ref/ncn_pytorch.py:12-41

Fixtures are data only (inputs and expected outputs, numpy .npz, no pickles).
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _inputs(batch, N, E, L, w_std, seed, dtype, xa_zero):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, N, E, generator=g, dtype=torch.float64)
    xa = torch.zeros(batch, N, E, dtype=torch.float64) if xa_zero else torch.randn(
        batch, N, E, generator=g, dtype=torch.float64)
    Ws = [torch.randn(2 * E, generator=g, dtype=torch.float64) * w_std for _ in range(L)]
    dyi = torch.randn(batch, N, E, generator=g, dtype=torch.float64)
    dya = torch.randn(batch, N, E, generator=g, dtype=torch.float64)
    # fp32 fixtures use the fp32 rounding of the same draws, so both precisions see "the same" inputs
    cast = lambda t: t.to(torch.float32).to(dtype)
    return cast(x), cast(xa), [cast(w) for w in Ws], cast(dyi), cast(dya)


def _run_net(net_cls, alpha, n, C, x, xa, Ws, dyi, dya):
    x = x.clone().requires_grad_()
    xa = xa.clone().requires_grad_()
    Ws = [w.clone().requires_grad_() for w in Ws]
    net = net_cls(alpha, "tanh", len(Ws), n, C, Ws)
    yi, ya = net(x, xa)
    torch.autograd.backward([yi, ya], [dyi, dya])
    out = {"yi": yi.detach(), "ya": ya.detach(), "dx": x.grad, "dxa": xa.grad}
    for l, w in enumerate(Ws):
        out[f"dW{l}"] = w.grad
    return out


def _case(name, ref, inv, *, batch, N, E, C, n, L, alpha, w_std, seed, xa_zero, run_inv):
    blob = {"meta": np.array([batch, N, E, C, n, L, seed, int(xa_zero)], dtype=np.int64),
            "alpha": np.array(alpha, dtype=np.float64)}
    for tag, dtype in (("f32", torch.float32), ("f64", torch.float64)):
        x, xa, Ws, dyi, dya = _inputs(batch, N, E, L, w_std, seed, dtype, xa_zero)
        if tag == "f32":
            blob.update({"x": x.numpy(), "xa": xa.numpy(), "dyi": dyi.numpy(), "dya": dya.numpy()})
            for l, w in enumerate(Ws):
                blob[f"W{l}"] = w.numpy()
        out = _run_net(ref.RefTorchNaive, alpha, n, C, x, xa, Ws, dyi, dya)
        for k, v in out.items():
            blob[f"ref_{tag}_{k}"] = v.numpy()
        if run_inv:
            out = _run_net(inv.RefInvTorchNaive, alpha, n, C, x, xa, Ws, dyi, dya)
            for k, v in out.items():
                blob[f"inv_{tag}_{k}"] = v.numpy()
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path}: {os.path.getsize(path)} bytes")


def _index_fixture(ref):
    rows = []
    for (N, n) in ((256, 2), (64, 4), (48, 3), (128, 16), (32, 32), (2048, 8)):
        m = N // n
        stages = sorted(set(list(range(0, min(12, m.bit_length() + 2))) + [m.bit_length() + 3]))
        for stage in stages:
            o = torch.arange(0, n, dtype=torch.long)
            for b in sorted({0, 1 % m, m // 2, m - 1, 5 % m}):
                idx = ref.group_pos_to_index_v2(N, n, stage, b, o)
                for oo in range(n):
                    rows.append((N, n, stage, b, oo, int(idx[oo])))
    arr = np.array(rows, dtype=np.int64)
    path = os.path.join(HERE, "index_map.npz")
    np.savez_compressed(path, rows=arr)
    print(f"wrote {path}: {arr.shape[0]} rows")


def _invert_fixture(inv):
    g = torch.Generator().manual_seed(7)
    n, Ec = 8, 6
    blob = {}
    for tag, dtype in (("f32", torch.float32), ("f64", torch.float64)):
        yi = torch.randn(n, Ec, generator=g, dtype=torch.float64).to(torch.float32).to(dtype)
        ya = torch.randn(n, Ec, generator=g, dtype=torch.float64).to(torch.float32).to(dtype)
        Wi = (0.4 * torch.randn(Ec, generator=g, dtype=torch.float64)).to(torch.float32).to(dtype)
        Wj = (0.4 * torch.randn(Ec, generator=g, dtype=torch.float64)).to(torch.float32).to(dtype)
        blob.update({f"{tag}_yi": yi.numpy(), f"{tag}_ya": ya.numpy(),
                     f"{tag}_Wi": Wi.numpy(), f"{tag}_Wj": Wj.numpy()})
        for j in (0, 3, 7):
            xi, xa = inv.NCNFunctionPytorch.invert(yi, ya, Wi, Wj, n, 0.9, "tanh", j)
            blob[f"{tag}_xi_j{j}"] = xi.numpy()
            blob[f"{tag}_xa_j{j}"] = xa.numpy()
    path = os.path.join(HERE, "invert_step.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path}")


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = _load(os.path.join(root, "torch_ref", "ncn_pytorch.py"), "ref_ncn_pytorch")
    inv = _load(os.path.join(root, "torch_ref", "ncn_pytorch_invertible.py"), "ref_ncn_pytorch_invertible")
    torch.set_num_threads(4)
    _index_fixture(ref)
    _invert_fixture(inv)
    # benchmark configuration 1: x [B=32, D=256], g=2, 8 stages  ->  [batch=1, N=256, E=32], 4 heads of 8
    _case("cfg1_n2_L8", ref, inv, batch=1, N=256, E=32, C=4, n=2, L=8, alpha=0.9,
          w_std=(1 / 2) ** 0.5, seed=0, xa_zero=True, run_inv=False)
    # multi-batch, multi-head, n=4, 3 stages, xa != 0, alpha != 0.9, both heads differ in W
    _case("small_n4_L3", ref, inv, batch=2, N=32, E=12, C=2, n=4, L=3, alpha=0.7,
          w_std=0.5, seed=1, xa_zero=False, run_inv=True)
    # the shape family the reference's own script exercises (n_cache == Ec), shrunk; wraps the stride (L > log2(m)+1)
    _case("bench_like_n8_L5", ref, inv, batch=1, N=64, E=16, C=2, n=8, L=5, alpha=0.9,
          w_std=0.5, seed=2, xa_zero=True, run_inv=True)
    # non power-of-two group size and odd head width
    _case("odd_n3_L3", ref, inv, batch=1, N=24, E=10, C=2, n=3, L=3, alpha=0.9,
          w_std=0.5, seed=3, xa_zero=False, run_inv=False)


if __name__ == "__main__":
    main()
