"""Seeded sweep over small random problems: every kernel path (register tiles, generic LDS kernel, multi-stage
passes, table / context-length builds) against the float64 oracle.  Shapes include n_cache = 1, n_cache = 64, one
feature per head, one group, one batch entry, group counts that are not powers of two."""
import random

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


def _cases(seed, count, acts=None):
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        n = rng.choice([1, 2, 2, 3, 4, 4, 5, 8, 8, 16, 16, 32, 64])
        ec = rng.choice([1, 3, 4, 4, 8, 8, 16, 16, 32, 32, 40, 64, 128])
        if ec == 128 and n not in (2, 4, 8, 16):
            continue                                   # no kernel for that pair (head width > 64 needs a register tile)
        C = rng.choice([1, 2, 4]) if ec <= 32 else rng.choice([1, 2])
        groups = rng.choice([1, 2, 3, 4, 6, 8, 16, 24, 32])
        if n * groups * ec * C > 1 << 17:
            continue
        batch = rng.choice([1, 2, 3, 5])
        L = rng.randint(1, 4 if n >= 8 else 6)
        first = rng.choice([0, 0, 1, 3])
        act = rng.choice([0, 0, 0, 2, -1, 3])
        out.append((batch, n * groups, ec * C, C, n, first, L, act if acts is None else acts[len(out) % len(acts)]))
    return out


def _one_feature_cases(seed, count):
    """Heads of one feature (E == n_head) on the group sizes and widths their register kernels exist for, and some
    they do not (E not a multiple of 4, n_cache not a power of two: generic kernels)."""
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        n = rng.choice([2, 2, 4, 4, 8, 16, 16, 32, 64, 3])
        E = rng.choice([4, 8, 12, 16, 20, 24, 32, 48, 64, 96, 128, 6])
        groups = rng.choice([1, 2, 3, 4, 6, 8, 16, 24, 32])
        if n * groups * E > 1 << 16:
            continue
        batch = rng.choice([1, 2, 3, 5])
        L = rng.randint(1, 4 if n >= 8 else 6)
        out.append((batch, n * groups, E, E, n, rng.choice([0, 0, 1, 3]), L, rng.choice([0, 0, 0, 2, -1, 3])))
    return out


# 16 of them: relu and leaky relu (codes 1 and 3) on inputs that stay away from the kink; the last 24: one feature per head
CASES = _cases(2024, 40) + _cases(7, 40) + _cases(11, 16, acts=(1, 3)) + _one_feature_cases(5, 24)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_N%d_E%d_C%d_n%d_s%d_L%d_a%d" % c)
def test_random_problem(M, case):
    batch, N, E, C, n, first, L, act = case
    alpha = 0.85
    if act in (1, 3):
        # relu / leaky relu: a float32 recomputation picks the other slope where |T| ~ 1e-7; inputs whose T keeps its
        # sign (positive in even batch entries, negative in odd ones) exercise both slopes and stay away from the kink
        x, xa, Ws, dy, dya = O.make_inputs_signed_regimes(batch, N, E, L, n, seed=sum(case) + 5)
    else:
        x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=sum(case) + 5, xa_zero=False)
    d = torch.float64
    ref = O.net_autograd(x.to(d), xa.to(d), [w.to(d) for w in Ws], dy.to(d), dya.to(d), alpha, n, C, activation=act,
                         first_stage=first)
    gx, gxa, gdy, gdya = x.cuda(), xa.cuda(), dy.cuda(), dya.cuda()
    W = torch.stack(Ws).cuda()
    amp_stage = (1 / 0.9) ** n
    # float32 rounding of the inversion grows like (1/m)^n per stage: 5x at n = 16, 29x at n = 32, 850x at n = 64
    # (where the reference's own check uses atol = 1e-2, grad_test_bench.py:161).  n <= 16, the group sizes of the
    # benchmark configurations, are held to 1e-5 whatever the amplification.  Above, the bounds are a margin over the
    # worst case measured on 370 shapes of this generator with 32 and 64 rows per group (30 seeds beyond the ones
    # below), per unit of amplification.  Gradients: 8.2e-7 at n = 32 (1.3e-6 on the sign-regime inputs of relu / leaky
    # relu), 1.2e-5 at n = 64 (1.5e-5).  Reconstructed inputs: 3.7e-6 at n = 32 (8.3e-6), and 0.073 absolute at n = 64
    # (0.15).
    signed = act in (1, 3)
    if n < 32:
        gtol, rtol = 1e-5, max(3e-5, 6e-6 * amp_stage)
    elif n < 64:
        gtol, rtol = (2e-6 if signed else 1.2e-6) * amp_stage, (1.2e-5 if signed else 6e-6) * amp_stage
    else:
        gtol, rtol = (2e-5 if signed else 1.6e-5) * amp_stage, (2e-1 if signed else 1e-1)
    # one call per stage, every stage saving its outputs
    outs, cx, cxa = [], gx, gxa
    for l in range(L):
        cx, cxa = M.forward_stages(cx, cxa, W[l], alpha, act, n, C, first + l, 1)
        outs.append((cx, cxa))
    assert O.rel_err(cx, ref[0]) < 1e-5 and O.rel_err(cxa, ref[1]) < 1e-5
    g, h = gdy, gdya
    worst_dw = worst_rec = 0.0
    for l in range(L - 1, -1, -1):
        xr, xar, g, h, dW = M.backward_stages(outs[l][0], outs[l][1], g, h, W[l], alpha, act, n, C, first + l, 1)
        prev = outs[l - 1] if l else (gx, gxa)
        worst_dw = max(worst_dw, O.rel_err(dW[0], ref[4][l]))
        worst_rec = max(worst_rec, O.rel_err(xr, prev[0]), O.rel_err(xar, prev[1]))
        assert O.rel_err(dW[0], ref[4][l]) < gtol, f"dW{l}"
        assert O.rel_err(xr, prev[0]) < rtol and O.rel_err(xar, prev[1]) < rtol
    if n >= 32:
        from conftest import record_errors
        record_errors("random_problem", n=n, act=act, amp=amp_stage, dW=worst_dw, rec=worst_rec,
                      dx=O.rel_err(g, ref[2]), dxa=O.rel_err(h, ref[3]))
    assert O.rel_err(g, ref[2]) < gtol and O.rel_err(h, ref[3]) < gtol
    # the same stages in one call (multi-stage passes where the shape allows), forward only compared tightly
    y, ya = M.forward_stages(gx, gxa, W, alpha, act, n, C, first, L)
    assert O.rel_err(y, ref[0]) < 1e-5 and O.rel_err(ya, ref[1]) < 1e-5
    if (1 / 0.9) ** (n * L) < 50:
        _, _, dx, dxa, dWs = M.backward_stages(y, ya, gdy, gdya, W, alpha, act, n, C, first, L)
        tol = max(1e-5, 2e-6 * (1 / 0.9) ** (n * L))
        assert O.rel_err(dx, ref[2]) < tol and O.rel_err(dxa, ref[3]) < tol
        for l in range(L):
            assert O.rel_err(dWs[l], ref[4][l]) < tol
    # a random table and ragged lengths through the indexed entry points
    gen = torch.Generator().manual_seed(sum(case))
    table = torch.randperm(N, generator=gen)
    lens = [int(v) for v in torch.randint(0, N + 1, (batch,), generator=gen)]
    iref = O.net_autograd_indexed(x.to(d), xa.to(d), [Ws[0].to(d)], dy.to(d), dya.to(d), alpha, n, C, [table], lens,
                                  activation=act)
    gt, gl = table.to(torch.int32).cuda(), torch.tensor(lens, dtype=torch.int32).cuda()
    iy, iya = M.forward_stages(gx, gxa, W[0], alpha, act, n, C, 0, 1, group_index=gt, ctx_len=gl)
    assert O.rel_err(iy, iref[0]) < 1e-5 and O.rel_err(iya, iref[1]) < 1e-5
    ixr, ixar, idx, idxa, idW = M.backward_stages(iy, iya, gdy, gdya, W[0], alpha, act, n, C, 0, 1, group_index=gt,
                                                  ctx_len=gl)
    assert O.rel_err(ixr, x) < rtol
    assert O.rel_err(idx, iref[2]) < gtol and O.rel_err(idxa, iref[3]) < gtol
    assert O.rel_err(idW[0], iref[4][0]) < gtol
    # the first levels of the radix-n grouping that N admits, without tables
    levels = 0
    while n > 1 and levels < L and N % n ** (levels + 1) == 0:
        levels += 1
    if levels:
        rtables = [O.radix_group_table(N, n, l) for l in range(levels)]
        rref = O.net_autograd_indexed(x.to(d), xa.to(d), [w.to(d) for w in Ws[:levels]], dy.to(d), dya.to(d), alpha, n, C,
                                      rtables, activation=act)
        ry, rya = M.forward_radix(gx, gxa, W[:levels], alpha, act, n, C, 0, levels)
        assert O.rel_err(ry, rref[0]) < 1e-5 and O.rel_err(rya, rref[1]) < 1e-5
        if (1 / 0.9) ** (n * levels) < 50:
            rxr, _, rdx, rdxa, rdW = M.backward_radix(ry, rya, gdy, gdya, W[:levels], alpha, act, n, C, 0, levels)
            tol = max(1e-5, 2e-6 * (1 / 0.9) ** (n * levels))
            assert O.rel_err(rdx, rref[2]) < tol and O.rel_err(rdxa, rref[3]) < tol
            # the reconstruction carries the rounding of every step it undoes: 1e-5 x (1/m)^(steps), as above
            assert O.rel_err(rxr, x) < max(3e-5, 1e-5 * (1 / 0.9) ** (n * levels))
            for l in range(levels):
                assert O.rel_err(rdW[l], rref[4][l]) < tol
