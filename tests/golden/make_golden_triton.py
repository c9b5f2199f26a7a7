#!/usr/bin/env python3
"""Writes tests/golden/triton_*.npz from the reference's Triton kernels, run by Triton's CPU interpreter.

Run once, in the development container only (the reference tree does not exist on the GPU box):

    python tests/golden/make_golden_triton.py [/root/reference]

Why.  torch_ref only knows tanh, and it has neither group tables nor context lengths, so the fixtures of
make_golden.py leave three things of the oracle without an independent statement:

  * the leaky-relu and linear activations (ncn_triton/ncn_triton.py:22-28, 101-106, 188-196), forward and the
    hand-written backward (:176-247);
  * grouping by a table of positions (ncn_triton/ncn_triton_old.py:66-71), with the radix-n tables that
    ncn_triton/group_tensors.py:8-18 defines;
  * one context length per batch entry (ncn_triton_old.py:64, 93-96): which groups run and, in the group a length
    cuts, which steps run.

The reference states them only as Triton kernels.  TRITON_INTERPRET=1 makes triton.jit run a kernel program by
program with numpy on CPU tensors, so the kernels' own text is what produces the numbers here; nothing of it is
kept, the fixtures are inputs and outputs only (numpy .npz, no pickles).

What the older kernel's outputs mean (read off ncn_triton_old.py, and visible in the numbers):
  * groups that start at or past the length are not touched: their rows of the outputs stay as torch.empty_like
    left them, so only live rows are recorded (`live` mask in the fixture) and the upstream gradient is zero elsewhere;
  * in the group a length cuts, the rows past the length read their position with a masked load (:66) whose
    fill is 0, so they alias position 0: they take part as ordinary rows and are stored over position 0.  The live
    rows never see them (a row's step only reads itself and the pivot, and only live rows are pivots), so the
    forward of live rows is well defined except at position 0; the backward sums over all rows of the group and
    reads what the forward left at position 0, so with a cut group it is an artefact -- unless position 0 is itself a
    dead row (a table that puts it in the last slot) and dead rows carry no upstream gradient: those cases are
    recorded forward and backward (`cutbwd*`).
  * xa is ignored and starts from zeros (:79): the fixtures pass zeros.
"""
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"   # before triton is imported

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ALPHA = 0.9


def _draw(gen, *shape, scale=1.0):
    return (torch.randn(*shape, generator=gen, dtype=torch.float64) * scale).to(torch.float32)


def _run(fn, x, xa, Ws, dyi, dya):
    x = x.clone().requires_grad_()
    xa = xa.clone().requires_grad_()
    Ws = [w.clone().requires_grad_() for w in Ws]
    yi, ya = fn(x, xa, Ws)
    torch.autograd.backward([yi, ya], [dyi.contiguous(), dya.contiguous()])
    out = {"yi": yi.detach(), "ya": ya.detach(), "dx": x.grad, "dxa": xa.grad}
    for l, w in enumerate(Ws):
        out[f"dW{l}"] = w.grad
    return {k: v.numpy().copy() for k, v in out.items()}


def activations(T):
    """One stage, forward + backward, per activation name and stage number; then a three-stage stack."""
    batch, N, E, C, n = 2, 32, 16, 2, 4
    blob = {"meta": np.array([batch, N, E, C, n], dtype=np.int64), "alpha": np.array(ALPHA)}
    gen = torch.Generator().manual_seed(2024)
    for act in ("tanh", "leaky-relu", "none"):
        for l in (0, 1, 3):
            x, xa = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
            W = _draw(gen, 2 * E, scale=0.3)
            dyi, dya = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
            out = _run(lambda a, b, ws: T.fused_ncn_triton(a, b, ws[0], ALPHA, act, C, n, l), x, xa, [W], dyi, dya)
            tag = f"{act}_l{l}_"
            blob.update({tag + "x": x.numpy(), tag + "xa": xa.numpy(), tag + "W": W.numpy(), tag + "dyi": dyi.numpy(),
                         tag + "dya": dya.numpy()})
            blob.update({tag + k: v for k, v in out.items()})
    # the stack class the reference's bench script builds (ncn_triton.py:395-417), leaky-relu, n_cache 2
    batch, N, E, C, n, L = 2, 16, 8, 2, 2, 3
    x, xa = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
    Ws = [_draw(gen, 2 * E, scale=0.4) for _ in range(L)]
    dyi, dya = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
    out = _run(lambda a, b, ws: T.NCNNetTestTriton(ALPHA, "leaky-relu", n, C, L, ws)(a, b), x, xa, Ws, dyi, dya)
    blob["net_meta"] = np.array([batch, N, E, C, n, L], dtype=np.int64)
    blob.update({"net_x": x.numpy(), "net_xa": xa.numpy(), "net_dyi": dyi.numpy(), "net_dya": dya.numpy()})
    for l, w in enumerate(Ws):
        blob[f"net_W{l}"] = w.numpy()
    blob.update({"net_" + k: v for k, v in out.items()})
    return blob


def headline_tile(T):
    """The headline shape's tile (groups of 16 rows, 4 heads of 32 features, tanh, 3 stages) on a short sequence:
    torch_ref's fixtures stop at groups of 8."""
    batch, N, E, C, n, L = 1, 64, 128, 4, 16, 3
    gen = torch.Generator().manual_seed(16)
    x, xa = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
    Ws = [_draw(gen, 2 * E, scale=0.25) for _ in range(L)]
    dyi, dya = _draw(gen, batch, N, E), _draw(gen, batch, N, E)
    out = _run(lambda a, b, ws: T.NCNNetTestTriton(ALPHA, "tanh", n, C, L, ws)(a, b), x, xa, Ws, dyi, dya)
    blob = {"meta": np.array([batch, N, E, C, n, L], dtype=np.int64), "alpha": np.array(ALPHA),
            "x": x.numpy(), "xa": xa.numpy(), "dyi": dyi.numpy(), "dya": dya.numpy()}
    for l, w in enumerate(Ws):
        blob[f"W{l}"] = w.numpy()
    blob.update(out)
    return blob


def radix_table(G, N, n, level):
    """Positions in (group, slot) order from the reference's digit split (group_tensors.py:8-18)."""
    strides = [n ** k for k in range(16)]
    table = [-1] * N
    for i in range(N):
        slot, group = G.extract_group_index(i, level, strides, n)
        table[group * n + slot] = i
    assert sorted(table) == list(range(N))
    return torch.tensor(table, dtype=torch.int32)


def tables_and_lengths(TO, G):
    """The older kernels: a table of positions and one context length per batch entry."""
    batch, N, E, C, n = 3, 32, 16, 2, 4
    blob = {"meta": np.array([batch, N, E, C, n], dtype=np.int64), "alpha": np.array(ALPHA)}
    gen = torch.Generator().manual_seed(77)
    scrambled = torch.randperm(N, generator=gen).to(torch.int32)     # any permutation is a legal table
    cases = []
    for level in (0, 1):
        cases.append((f"radix{level}", radix_table(G, N, n, level)))
    cases.append(("scrambled", scrambled))
    k = 0
    for tname, table in cases:
        blob[f"table_{tname}"] = table.numpy()
        # whole groups only: forward and backward are well defined on the live rows
        for lens in ([N, N, N], [8, 20, N], [0, 4, 28]):
            for act in ("tanh", "leaky-relu"):
                x = _draw(gen, batch, N, E)
                xa = torch.zeros(batch, N, E)
                W = _draw(gen, 2 * E, scale=0.3)
                ctx = torch.tensor(lens, dtype=torch.int32)
                live = torch.zeros(batch, N, dtype=torch.bool)
                for b in range(batch):
                    live[b, table[:lens[b]].long()] = True
                dyi = _draw(gen, batch, N, E) * live[:, :, None]
                dya = _draw(gen, batch, N, E) * live[:, :, None]
                out = _run(lambda a, b_, ws: TO.fused_chunk_linear_ncn(a, b_, ws[0], table, ctx, ALPHA, act, C, n, 0),
                           x, xa, [W], dyi, dya)
                tag = f"whole{k}_"
                k += 1
                blob[tag + "table"] = np.array(tname)
                blob[tag + "act"] = np.array(act)
                blob.update({tag + "ctx_len": ctx.numpy(), tag + "live": live.numpy(), tag + "x": x.numpy(),
                             tag + "W": W.numpy(), tag + "dyi": dyi.numpy(), tag + "dya": dya.numpy()})
                for key, v in out.items():
                    # rows the kernels never wrote hold whatever the allocator left: keep the live rows only
                    if key in ("yi", "ya", "dx", "dxa"):
                        v = np.where(live.numpy()[:, :, None], v, 0.0).astype(np.float32)
                    blob[tag + key] = v
    blob["n_whole"] = np.array(k)
    # lengths that cut a group: forward only, live rows only, position 0 excluded (see the module docstring)
    k = 0
    for tname, table in cases:
        for lens in ([7, 13, 30], [1, 18, 31]):
            x = _draw(gen, batch, N, E)
            W = _draw(gen, 2 * E, scale=0.3)
            ctx = torch.tensor(lens, dtype=torch.int32)
            live = torch.zeros(batch, N, dtype=torch.bool)
            for b in range(batch):
                live[b, table[:lens[b]].long()] = True
            check = live.clone()
            check[:, 0] = False
            with torch.no_grad():
                yi, ya = TO.fused_chunk_linear_ncn(x, torch.zeros_like(x), W, table, ctx, ALPHA, "tanh", C, n, 0)
            tag = f"cut{k}_"
            k += 1
            m = check.numpy()[:, :, None]
            blob[tag + "table"] = np.array(tname)
            blob.update({tag + "ctx_len": ctx.numpy(), tag + "check": check.numpy(), tag + "x": x.numpy(),
                         tag + "W": W.numpy(), tag + "yi": np.where(m, yi.numpy(), 0.0).astype(np.float32),
                         tag + "ya": np.where(m, ya.numpy(), 0.0).astype(np.float32)})
    blob["n_cut"] = np.array(k)
    # lengths that cut a group, forward AND backward: with position 0 in the table's last slot it is a dead row for
    # every length below N, so the rows that alias it disturb nobody live, and with no upstream gradient on dead rows
    # (u = 0, r = 0 for them) they add nothing to the pivot row's gradient or to dW: the kernel's backward of the cut
    # group is then well defined on the live rows
    k = 0
    for trial in range(2):
        perm = torch.randperm(N, generator=gen)
        at = int((perm == 0).nonzero()[0])
        perm[at], perm[N - 1] = perm[N - 1].clone(), perm[at].clone()
        table = perm.to(torch.int32)
        for lens in ([7, 13, 30], [1, 18, 31], [5, 5, 22]):
            x = _draw(gen, batch, N, E)
            W = _draw(gen, 2 * E, scale=0.3)
            ctx = torch.tensor(lens, dtype=torch.int32)
            live = torch.zeros(batch, N, dtype=torch.bool)
            for b in range(batch):
                live[b, table[:lens[b]].long()] = True
            dyi = _draw(gen, batch, N, E) * live[:, :, None]
            dya = _draw(gen, batch, N, E) * live[:, :, None]
            act = "tanh" if k % 2 == 0 else "leaky-relu"
            out = _run(lambda a, b_, ws: TO.fused_chunk_linear_ncn(a, b_, ws[0], table, ctx, ALPHA, act, C, n, 0),
                       x, torch.zeros(batch, N, E), [W], dyi, dya)
            tag = f"cutbwd{k}_"
            k += 1
            blob[tag + "act"] = np.array(act)
            blob.update({tag + "table": table.numpy(), tag + "ctx_len": ctx.numpy(), tag + "live": live.numpy(),
                         tag + "x": x.numpy(), tag + "W": W.numpy(), tag + "dyi": dyi.numpy(), tag + "dya": dya.numpy()})
            for key, v in out.items():
                if key in ("yi", "ya", "dx", "dxa"):
                    v = np.where(live.numpy()[:, :, None], v, 0.0).astype(np.float32)
                blob[tag + key] = v
    blob["n_cutbwd"] = np.array(k)
    return blob


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, ref_root)
    from ncn_triton import group_tensors as G
    from ncn_triton import ncn_triton as T
    from ncn_triton import ncn_triton_old as TO
    np.savez_compressed(os.path.join(HERE, "triton_activations.npz"), **activations(T))
    np.savez_compressed(os.path.join(HERE, "triton_tables_lengths.npz"), **tables_and_lengths(TO, G))
    np.savez_compressed(os.path.join(HERE, "triton_headline_tile.npz"), **headline_tile(T))
    print("wrote triton_activations.npz, triton_tables_lengths.npz, triton_headline_tile.npz")


if __name__ == "__main__":
    main()
