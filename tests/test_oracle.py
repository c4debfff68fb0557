"""CPU tests that pin the oracle (the reference ships no tests or fixtures for this path).

Each check is chosen so that a plausible mistake fails it: a dropped term (row sums),
a wrong index or off-by-one in the cumulative sum (closed form 2^-(i-j), brute force),
a wrong sign (finite differences), a transposed operand (gradients vs the C brute
force, dk vs dq shapes on asymmetric data).
"""
import math

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import sb_oracle as O
from helpers import randn


def test_closed_form_zero_logits():
    # q = 0 -> beta = 1/2 everywhere -> A_ij = 2^-(i-j), rem_i = 2^-i  (strict causal)
    T, D = 12, 4
    q = torch.zeros(1, 1, T, D, dtype=torch.float64)
    k = randn((1, 1, T, D), 1, dtype=torch.float64)
    v = torch.eye(T, dtype=torch.float64)[None, None]        # o rows = attention rows
    o, rem = O.sb_attn_oracle(q, k, v, compute_dtype=torch.float64)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    expect = torch.where(j < i, 2.0 ** (-(i - j).double()), torch.zeros((), dtype=torch.float64))
    assert torch.allclose(o[0, 0], expect, atol=1e-14)
    assert torch.allclose(rem[0, 0], 2.0 ** (-torch.arange(T).double()), atol=1e-14)


def test_closed_form_attend_current():
    T, D = 9, 4
    q = torch.zeros(1, 1, T, D, dtype=torch.float64)
    k = randn((1, 1, T, D), 2, dtype=torch.float64)
    v = torch.eye(T, dtype=torch.float64)[None, None]
    o, rem = O.sb_attn_oracle(q, k, v, attend_current=True, compute_dtype=torch.float64)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    expect = torch.where(j <= i, 2.0 ** (-(i - j + 1).double()), torch.zeros((), dtype=torch.float64))
    assert torch.allclose(o[0, 0], expect, atol=1e-14)
    assert torch.allclose(rem[0, 0], 2.0 ** (-(torch.arange(T) + 1).double()), atol=1e-14)


def test_saturated_limits():
    T, D = 6, 2
    k = torch.ones(1, 1, T, D, dtype=torch.float64)
    v = torch.eye(T, dtype=torch.float64)[None, None][..., :T]
    # z -> +inf: all mass on the nearest key, rem -> 0
    o, rem = O.sb_attn_oracle(40 * torch.ones(1, 1, T, D, dtype=torch.float64), k, v,
                              inv_temp=1.0, compute_dtype=torch.float64)
    assert torch.allclose(o[0, 0, 1:], torch.eye(T, dtype=torch.float64)[:-1], atol=1e-12)
    assert torch.allclose(rem[0, 0, 1:], torch.zeros(T - 1, dtype=torch.float64), atol=1e-12)
    assert rem[0, 0, 0] == 1 and o[0, 0, 0].abs().max() == 0     # row 0 sees no key
    # z -> -inf: nothing attended, rem -> 1
    o, rem = O.sb_attn_oracle(-40 * torch.ones(1, 1, T, D, dtype=torch.float64), k, v,
                              inv_temp=1.0, compute_dtype=torch.float64)
    assert o.abs().max() < 1e-12 and torch.allclose(rem, torch.ones_like(rem), atol=1e-12)


@pytest.mark.parametrize("attend_current", [False, True])
def test_literal_einsum_form_equals_cumsum_form(attend_current):
    # sb_ref.py's statement (mask + cum_weight einsum) vs the O(T^2) form used everywhere else
    B, H, T, D = 2, 3, 33, 8
    q, k, v = (randn((B, H, T, D), s, dtype=torch.float64) for s in (3, 4, 5))
    mask = O.causal_mask(T, attend_current)
    cw = O.cum_weight(T, torch.float64)
    o1, r1 = O.stickbreaking_literal(q, k, v, mask, cw)
    o2, r2 = O.sb_attn_oracle(q, k, v, attend_current=attend_current, compute_dtype=torch.float64)
    # the literal form casts logits to float32 (sb_ref.py:16), hence 1e-6 and not 1e-12
    assert torch.allclose(o1, o2, atol=2e-6)
    assert torch.allclose(r1, r2, atol=2e-6)
    o3, r3 = O.sb_attn_oracle_rem_by_sum(q, k, v, attend_current=attend_current)
    assert torch.allclose(r3, r2, atol=1e-12) and torch.allclose(o3, o2, atol=1e-14)


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("T,D,scale", [(1, 4, 0.5), (7, 3, 1.0), (16, 8, 0.35), (40, 16, 0.25)])
def test_forward_vs_c_bruteforce(T, D, scale, attend_current):
    q, k, v = (randn((T, D), s, scale=1.5, dtype=torch.float64) for s in (10, 11, 12))
    o_c, rem_c, A_c = c_oracle.forward(q.numpy(), k.numpy(), v.numpy(), scale, attend_current)
    o, rem = O.sb_attn_oracle(q[None, None], k[None, None], v[None, None], inv_temp=scale,
                              attend_current=attend_current, compute_dtype=torch.float64)
    assert np.allclose(o[0, 0].numpy(), o_c, atol=1e-12)
    assert np.allclose(rem[0, 0].numpy(), rem_c, atol=1e-12)
    # invariants of the brute force itself
    assert (A_c >= 0).all() and (A_c <= 1).all()
    assert np.allclose(A_c.sum(-1) + rem_c, 1.0, atol=1e-14)
    assert np.all(np.triu(A_c, 1 if attend_current else 0) == 0)


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("T,D", [(5, 3), (12, 4), (24, 8)])
def test_gradients_autograd_vs_c_bruteforce_vs_closed_form(T, D, attend_current):
    scale = 0.6
    q, k, v, do = (randn((T, D), s, dtype=torch.float64) for s in (20, 21, 22, 23))
    drem = randn((T,), 24, dtype=torch.float64)
    _, _, dq, dk, dv = O.sb_attn_grads_oracle(q[None, None], k[None, None], v[None, None], do[None, None],
                                               drem[None, None], inv_temp=scale,
                                               attend_current=attend_current,
                                               compute_dtype=torch.float64)
    dq_c, dk_c, dv_c = c_oracle.backward(q.numpy(), k.numpy(), v.numpy(), do.numpy(), drem.numpy(),
                                         scale, attend_current)
    for a, b in ((dq, dq_c), (dk, dk_c), (dv, dv_c)):
        assert np.allclose(a[0, 0].numpy(), b, atol=1e-11)
    # the algebra the kernels implement (g, prefix sum, beta) gives the same numbers
    dq2, dk2, dv2 = O.sb_attn_bwd_closed_form(q, k, v, do, drem, inv_temp=scale,
                                              attend_current=attend_current)
    for a, b in ((dq2, dq_c), (dk2, dk_c), (dv2, dv_c)):
        assert np.allclose(a.numpy(), b, atol=1e-11)


def test_gradients_finite_differences():
    T, D, scale = 6, 3, 0.7
    q, k, v, do = (randn((T, D), s, dtype=torch.float64) for s in (30, 31, 32, 33))
    drem = randn((T,), 34, dtype=torch.float64)

    def loss(qq, kk, vv):
        o, rem, _ = c_oracle.forward(qq, kk, vv, scale, False)
        return float((o * do.numpy()).sum() + (rem * drem.numpy()).sum())

    dq_c, dk_c, dv_c = c_oracle.backward(q.numpy(), k.numpy(), v.numpy(), do.numpy(), drem.numpy(), scale)
    eps = 1e-6
    for which, grad in enumerate((dq_c, dk_c, dv_c)):
        for idx in [(0, 0), (2, 1), (5, 2), (3, 0)]:
            args = [q.numpy().copy(), k.numpy().copy(), v.numpy().copy()]
            args[which][idx] += eps
            up = loss(*args)
            args[which][idx] -= 2 * eps
            dn = loss(*args)
            assert abs((up - dn) / (2 * eps) - grad[idx]) < 1e-7


def test_gradcheck_torch_restatement():
    T, D = 6, 3
    q, k, v = (randn((1, 1, T, D), s, dtype=torch.float64).requires_grad_(True) for s in (40, 41, 42))
    assert torch.autograd.gradcheck(
        lambda a, b, c: O.sb_attn_oracle(a, b, c, inv_temp=0.8, compute_dtype=torch.float64), (q, k, v))


def test_row_sum_identity_of_g():
    # sum_j g_ij = dO_i.o_i - drem_i (1 - rem_i): what a one-sweep backward may rely on
    T, D = 20, 8
    q, k, v, do = (randn((T, D), s, dtype=torch.float64) for s in (50, 51, 52, 53))
    drem = randn((T,), 54, dtype=torch.float64)
    o, rem, A = c_oracle.forward(q.numpy(), k.numpy(), v.numpy(), 0.5)
    g = A * (do.numpy() @ v.numpy().T - drem.numpy()[:, None])
    assert np.allclose(g.sum(-1), (do.numpy() * o).sum(-1) - drem.numpy() * (1 - rem), atol=1e-13)


@pytest.mark.parametrize("attend_current", [False, True])
def test_varlen_is_block_diagonal(attend_current):
    H, D = 2, 8
    lens = [5, 1, 17, 9]
    N = sum(lens)
    cu = torch.tensor([0, 5, 6, 23, 32])
    q, k, v = (randn((H, N, D), s, dtype=torch.float64) for s in (60, 61, 62))
    o, rem = O.sb_attn_varlen_oracle(q, k, v, cu, attend_current=attend_current, compute_dtype=torch.float64)
    start = 0
    for L in lens:
        for h in range(H):
            o_c, rem_c, _ = c_oracle.forward(q[h, start:start + L].numpy(), k[h, start:start + L].numpy(),
                                             v[h, start:start + L].numpy(), 1 / math.sqrt(D), attend_current)
            assert np.allclose(o[h, start:start + L].numpy(), o_c, atol=1e-12)
            assert np.allclose(rem[h, start:start + L].numpy(), rem_c, atol=1e-12)
        start += L
    # zero_start=False takes the document ends only
    o2, rem2 = O.sb_attn_varlen_oracle(q, k, v, cu[1:], zero_start=False, attend_current=attend_current,
                                       compute_dtype=torch.float64)
    assert torch.equal(o, o2) and torch.equal(rem, rem2)


def test_attend_current_relation_to_strict():
    # adding the diagonal key scales every A_ij (j<i) and rem_i by (1 - beta_ii)
    T, D = 15, 4
    q, k, v = (randn((T, D), s, dtype=torch.float64) for s in (70, 71, 72))
    s = 0.5
    _, rem0, A0 = c_oracle.forward(q.numpy(), k.numpy(), v.numpy(), s, False)
    _, rem1, A1 = c_oracle.forward(q.numpy(), k.numpy(), v.numpy(), s, True)
    beta_ii = 1 / (1 + np.exp(-s * (q.numpy() * k.numpy()).sum(-1)))
    assert np.allclose(np.tril(A1, -1), np.tril(A0, -1) * (1 - beta_ii)[:, None], atol=1e-14)
    assert np.allclose(np.diag(A1), beta_ii, atol=1e-14)
    assert np.allclose(rem1, rem0 * (1 - beta_ii), atol=1e-14)


def test_config1_shape_fp32_matches_fp64():
    # benchmark configuration 1 (B=2,H=4,T=512,d=64, N(0,1), scale 1/8): the fp32 oracle that the
    # 1e-4 GPU tolerance is measured against is itself within 1e-5 of float64
    q, k, v = (randn((2, 4, 512, 64), s) for s in (0, 1, 2))
    o32, r32 = O.sb_attn_oracle(q, k, v)
    o64, r64 = O.sb_attn_oracle(q, k, v, compute_dtype=torch.float64)
    assert (o32.double() - o64).abs().max() < 1e-5
    assert (r32.double() - r64).abs().max() < 1e-5
    assert o32.shape == (2, 4, 512, 64) and r32.shape == (2, 4, 512)
