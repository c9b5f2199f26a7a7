"""Pins of the oracle's table-grouped / context-length stage (oracle.stage_forward_indexed) and of the tables.

The reference states this variant only as Triton kernels (ncn_triton/ncn_triton_old.py:53-260) that cannot run here,
so the pins are: reduction to the pinned stage_forward (stride table, full lengths), literal loops on the group a
length cuts, the digit definition of the radix tables (ncn_triton/group_tensors.py:8-18) by brute force, and
inverse round trips.  The product's own table helpers (ncn_cuda_amd.chunk_linear) are checked against the same.
"""
import pytest
import torch

from oracle import ncn_oracle as O

D = torch.float64


def _rand(*shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=D) * scale


@pytest.mark.parametrize("stage", [0, 1, 2, 3, 5])
def test_stride_table_reproduces_pinned_stage(stage):
    B, N, E, C, n = 2, 24, 8, 2, 4
    x, xa, W = _rand(B, N, E, seed=1), _rand(B, N, E, seed=2), _rand(2 * E, seed=3, scale=0.3)
    want = O.stage_forward(x, xa, W, 0.8, n, C, stage)
    got = O.stage_forward_indexed(x, xa, W, 0.8, n, C, O.stride_group_table(N, n, stage))
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    full = O.stage_forward_indexed(x, xa, W, 0.8, n, C, O.stride_group_table(N, n, stage), ctx_len=[N, N + 7])
    assert torch.equal(full[0], want[0]) and torch.equal(full[1], want[1])


def test_context_length_by_literal_loops():
    """Identity table, lengths 0, 5, 8, 11 of N = 12 with n = 4, one head: groups below the length run 4 steps,
    the cut group runs `rem` steps on `rem` rows (ncn_triton_old.py:93-96), everything else passes through."""
    N, E, n, alpha, m = 12, 3, 4, 0.7, 0.9
    lens = [0, 5, 8, 11]
    x, xa, W = _rand(len(lens), N, E, seed=5), _rand(len(lens), N, E, seed=6), _rand(2 * E, seed=7, scale=0.4)
    y, ya = O.stage_forward_indexed(x, xa, W, alpha, n, 1, torch.arange(N), ctx_len=lens, m=m)
    Wi, Wj = W[:E], W[E:]
    for b, ln in enumerate(lens):
        r = [x[b, p].clone() for p in range(N)]
        a = [xa[b, p].clone() for p in range(N)]
        for g in range(N // n):
            rows = max(0, min(n, ln - g * n))
            idx = list(range(g * n, g * n + rows))
            for j in range(rows):
                xj = r[idx[j]]
                e = torch.dot(xj, Wj)
                nr, na = {}, {}
                for i in idx:
                    s = torch.dot(r[i], Wi) + e
                    F = torch.tanh(alpha * r[i] + (1 - alpha) * s * xj)
                    na[i] = m * a[i] + (1 - m) * F
                    nr[i] = m * r[i] + (1 - m) * na[i]
                for i in idx:
                    r[i], a[i] = nr[i], na[i]
        assert torch.allclose(y[b], torch.stack(r), atol=1e-14)
        assert torch.allclose(ya[b], torch.stack(a), atol=1e-14)
        assert torch.equal(y[b, ln:], x[b, ln:]) and torch.equal(ya[b, ln:], xa[b, ln:])


def test_dead_rows_follow_table_order_not_position():
    """With a non-trivial table the live slots are the first ctx_len entries of the table."""
    N, E, n = 16, 4, 2
    table = O.radix_group_table(N, n, 2)
    x, xa, W = _rand(1, N, E, seed=8), _rand(1, N, E, seed=9), _rand(2 * E, seed=10, scale=0.3)
    y, ya = O.stage_forward_indexed(x, xa, W, 0.9, n, 2, table, ctx_len=[6])
    dead = table[6:]
    assert torch.equal(y[0, dead], x[0, dead]) and torch.equal(ya[0, dead], xa[0, dead])
    live = table[:6]
    assert (y[0, live] != x[0, live]).all()


@pytest.mark.parametrize("N,n,level", [(16, 2, 0), (16, 2, 3), (27, 3, 1), (64, 4, 2), (48, 4, 1)])
def test_radix_table_is_the_digit_grouping(N, n, level):
    """Brute force over the definition of group_tensors.py:8-18."""
    table = O.radix_group_table(N, n, level)
    assert sorted(table.tolist()) == list(range(N))
    stride = n ** level
    for g in range(N // n):
        members = table[g * n:(g + 1) * n].tolist()
        for slot, i in enumerate(members):
            assert (i // stride) % n == slot                               # the digit at `level` is the slot
            assert i % stride + (i // (n * stride)) * stride == g          # the other digits number the group
        assert len({i - slot * stride for slot, i in enumerate(members)}) == 1   # they differ in that digit only


def test_radix_level0_is_stage0_and_hand_values():
    assert torch.equal(O.radix_group_table(32, 4, 0), O.stride_group_table(32, 4, 0))
    assert O.radix_group_table(16, 2, 1).tolist() == [0, 2, 1, 3, 4, 6, 5, 7, 8, 10, 9, 11, 12, 14, 13, 15]
    assert O.radix_group_table(27, 3, 1)[:9].tolist() == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    with pytest.raises(ValueError):
        O.radix_group_table(24, 4, 2)


def test_product_table_helpers_match():
    from ncn_cuda_amd import chunk_linear as CL
    for N, n, l in [(24, 4, 0), (24, 4, 3), (256, 2, 7), (36, 3, 4)]:
        assert torch.equal(CL.stride_group_table(N, n, l).long(), O.stride_group_table(N, n, l))
        for g, o in [(0, 0), (1, n - 1), (N // n - 1, 1 % n)]:
            assert int(CL.stride_group_table(N, n, l)[g * n + o]) == O.group_pos_to_index(N, n, l, g, o)
    for N, n, l in [(16, 2, 3), (27, 3, 1), (64, 4, 2), (48, 4, 1)]:
        assert torch.equal(CL.radix_group_table(N, n, l).long(), O.radix_group_table(N, n, l))
    with pytest.raises(ValueError):
        CL.radix_group_table(24, 4, 2)
    with pytest.raises(ValueError):
        CL.stride_group_table(10, 4, 0)


def test_indexed_inverse_round_trip_and_autograd_of_dead_rows():
    B, N, E, C, n, L = 2, 32, 8, 2, 4, 3
    x, xa = _rand(B, N, E, seed=11), _rand(B, N, E, seed=12)
    Ws = [_rand(2 * E, seed=20 + l, scale=0.3) for l in range(L)]
    tables = [O.radix_group_table(N, n, l % 2) for l in range(L)]
    lens = [13, 32]
    y, ya = O.net_forward_indexed(x, xa, Ws, 0.8, n, C, tables, lens)
    xi, xai = O.net_inverse_indexed(y, ya, Ws, 0.8, n, C, tables, lens)
    assert O.rel_err(xi, x) < 1e-12 and O.rel_err(xai, xa) < 1e-12
    dy, dya = _rand(B, N, E, seed=13), _rand(B, N, E, seed=14)
    _, _, dx, dxa, dWs = O.net_autograd_indexed(x, xa, Ws, dy, dya, 0.8, n, C, tables, lens)
    # a row that is dead in every stage passes its gradient through untouched
    dead = sorted(set(range(N)) - set().union(*[set(t[:13].tolist()) for t in tables]))
    assert dead
    assert torch.equal(dx[0, dead], dy[0, dead]) and torch.equal(dxa[0, dead], dya[0, dead])
    # dW is the sum of the per-batch-entry gradients (each entry has its own length)
    parts = [O.net_autograd_indexed(x[b:b + 1], xa[b:b + 1], Ws, dy[b:b + 1], dya[b:b + 1], 0.8, n, C, tables,
                                    lens[b:b + 1])[4] for b in range(B)]
    for l in range(L):
        assert O.rel_err(parts[0][l] + parts[1][l], dWs[l]) < 1e-12
