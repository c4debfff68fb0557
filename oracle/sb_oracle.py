"""CPU oracle for stick-breaking attention.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain PyTorch on the CPU, the algorithm of the reference
operator.  It is the checker that the HIP kernels are compared against; nothing in
the shipped package imports it.  Only tests, the smoke check and the benchmark's
``cpu_baseline`` leg may call it.

Reference lines each function follows (paths relative to the reference tree):

* ``stickbreaking_literal``  -- custom_models/sba/stickbreaking_attention/sb_ref.py:8-25
  (same statement order: logits, fp32 cast, log_z / log_beta with masked_fill,
  einsum with ``cum_weight``, exp, ``att @ v`` and ``1 - att.sum(-1)``).
* ``causal_mask`` / ``cum_weight``  -- the two inputs sb_ref.py:8 takes but the reference
  never builds; derived from the kernel's mask rule
  (sb_varlen/sb_varlen_fwd.py:48-51: strict ``M > N``, or ``M >= N`` when
  ``attend_current``) and from ``re_cum[i,k] = sum_{j>k} log_beta[i,j]`` (sb_ref.py:21-22).
* ``sb_attn_oracle``  -- same mathematics in O(T^2) memory-light form: a reversed
  cumulative sum instead of the T x T x T einsum; signature and defaults of
  sb_attn/__init__.py:57-64 (``inv_temp=None`` -> 1/sqrt(d), returns ``(o, rem)``).
* ``sb_attn_varlen_oracle``  -- sb_varlen/__init__.py:71-82 (``[H, sumT, D]`` packed
  layout, ``cu_seqlens`` with a leading 0 when ``zero_start``); every document is an
  independent dense problem (sb_varlen_fwd.py:280-285 computes per-document offsets).
* ``sb_attn_grads_oracle``  -- gradients by torch.autograd through the restatement; the
  closed form they must equal is sb_varlen_bwd.py:416-430
  (``g = A*(dO.v - drem)``, ``dz = g - beta*cumsum(g)``).

Pinning status: the reference ships no tests, fixtures or golden vectors for this path,
so the oracle is pinned by (tests/test_oracle.py): closed forms (q = 0 gives
A_ij = 2^-(i-j), rem_i = 2^-i), the identity sum_j A_ij + rem_i = 1, an independent
float64 brute-force evaluation of the product formula written in C (oracle/sb_oracle.c,
hand-derived gradients), central finite differences, equality of the literal einsum form
with the cumulative-sum form, the block-diagonal property of the packed layout, and the
golden vectors of tests/golden (the product formula and central differences of the loss in
50-digit arithmetic, tests/golden/make_vectors.py; reproduced to 1e-12 in tests/test_golden.py).
The one behaviour none of these pins is sb_ref.py's rounding order when it is *run in
bf16* (log_z / log_beta cast back to bf16 before the einsum): "parity unpinned" for
that; all tolerances here are against the oracle evaluated in fp32/fp64 on the same
(bf16-rounded) inputs, where that rounding order plays no part.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


def causal_mask(T: int, attend_current: bool = False, device=None) -> torch.Tensor:
    """``mask[i, j]`` is True where key j is NOT visible to query i."""
    return torch.ones(T, T, dtype=torch.bool, device=device).triu(1 if attend_current else 0)


def cum_weight(T: int, dtype=torch.float32, device=None) -> torch.Tensor:
    """``cum_weight[j, k] = 1`` where j > k, so ``(log_beta @ cum_weight)[i, k]`` sums j > k."""
    return torch.ones(T, T, dtype=dtype, device=device).tril(-1)


def stickbreaking_literal(q, k, v, mask, cum_weight):
    """Literal dense form (sb_ref.py:8-25); fixed scale 1/sqrt(d); O(T^3) einsum."""
    logits = (q @ k.transpose(-1, -2)) / math.sqrt(q.shape[-1])
    original_dtype = logits.dtype
    logits = logits.float()
    log_z = F.logsigmoid(logits).masked_fill(mask, -1e5).to(original_dtype)
    log_beta = F.logsigmoid(-logits).masked_fill(mask, 0).to(original_dtype)
    re_cum_log_beta = torch.einsum("bhij,jk->bhik", log_beta, cum_weight.to(log_beta))
    log_att = log_z + re_cum_log_beta
    att = log_att.exp()
    return att @ v, 1 - att.sum(dim=-1)


def _attention_matrix(q, k, inv_temp: float, attend_current: bool, compute_dtype):
    """A[..., i, j] and rem[..., i] for one dense problem; last two dims are [T, D]."""
    T = q.shape[-2]
    logits = (q.to(compute_dtype) @ k.to(compute_dtype).transpose(-1, -2)) * inv_temp
    mask = causal_mask(T, attend_current, device=q.device)
    log_z = F.logsigmoid(logits)
    log_beta = F.logsigmoid(-logits).masked_fill(mask, 0.0)
    # re_cum[i, j] = sum_{k > j} log_beta[i, k]   (exclusive reversed cumulative sum)
    incl = log_beta.flip(-1).cumsum(-1).flip(-1)
    re_cum = incl - log_beta
    att = (log_z + re_cum).exp().masked_fill(mask, 0.0)
    # rem_i = prod_k (1 - beta_ik) = exp(sum_k log_beta_ik); equals 1 - sum_j att_ij
    rem = incl[..., 0].exp()
    return att, rem


def sb_attn_oracle(q, k, v, inv_temp: Optional[float] = None, zero_start: bool = True,
                   attend_current: bool = False, compute_dtype=torch.float32
                   ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dense ``[B, H, T, D]`` (or any leading dims) stick-breaking attention -> (o, rem).

    Evaluated in ``compute_dtype`` on the given (possibly bf16-rounded) inputs; outputs are
    returned in ``compute_dtype`` so callers choose what to compare against.
    """
    if inv_temp is None:
        inv_temp = 1.0 / math.sqrt(q.shape[-1])
    att, rem = _attention_matrix(q, k, inv_temp, attend_current, compute_dtype)
    return att @ v.to(compute_dtype), rem


def sb_attn_oracle_rem_by_sum(q, k, v, inv_temp=None, attend_current=False,
                              compute_dtype=torch.float64):
    """Same as sb_attn_oracle but rem = 1 - sum_j A_ij exactly as sb_ref.py:25 writes it."""
    if inv_temp is None:
        inv_temp = 1.0 / math.sqrt(q.shape[-1])
    att, _ = _attention_matrix(q, k, inv_temp, attend_current, compute_dtype)
    return att @ v.to(compute_dtype), 1 - att.sum(-1)


def sb_attn_varlen_oracle(q, k, v, cu_seqlens, max_seqlens: Optional[int] = None,
                          inv_temp: Optional[float] = None, zero_start: bool = True,
                          attend_current: bool = False, compute_dtype=torch.float32):
    """Packed ``[H, sumT, D]`` layout; documents delimited by ``cu_seqlens``."""
    cu = [int(x) for x in cu_seqlens]
    if zero_start:
        assert cu[0] == 0
        cu = cu[1:]
    if inv_temp is None:
        inv_temp = 1.0 / math.sqrt(q.shape[-1])
    H, N, D = q.shape
    o = torch.zeros(H, N, v.shape[-1], dtype=compute_dtype)
    rem = torch.ones(H, N, dtype=compute_dtype)
    start = 0
    outs_o, outs_r = [], []
    for end in cu:
        if end > start:
            oo, rr = sb_attn_oracle(q[:, start:end], k[:, start:end], v[:, start:end],
                                    inv_temp=inv_temp, attend_current=attend_current,
                                    compute_dtype=compute_dtype)
            outs_o.append(oo)
            outs_r.append(rr)
        start = end
    if outs_o:
        o = torch.cat(outs_o, dim=1)
        rem = torch.cat(outs_r, dim=1)
    return o, rem


def sb_attn_grads_oracle(q, k, v, do, drem=None, inv_temp=None, attend_current=False,
                         cu_seqlens: Optional[Sequence[int]] = None,
                         compute_dtype=torch.float32):
    """(o, rem, dq, dk, dv) by autograd through the restatement.

    ``do`` / ``drem`` are the upstream gradients of ``o`` / ``rem``.  With ``cu_seqlens``
    (leading 0 included) the packed layout is used.
    """
    qq = q.detach().to(compute_dtype).requires_grad_(True)
    kk = k.detach().to(compute_dtype).requires_grad_(True)
    vv = v.detach().to(compute_dtype).requires_grad_(True)
    if cu_seqlens is None:
        o, rem = sb_attn_oracle(qq, kk, vv, inv_temp=inv_temp, attend_current=attend_current,
                                compute_dtype=compute_dtype)
    else:
        o, rem = sb_attn_varlen_oracle(qq, kk, vv, cu_seqlens, inv_temp=inv_temp,
                                       attend_current=attend_current,
                                       compute_dtype=compute_dtype)
    loss = (o * do.to(compute_dtype)).sum()
    if drem is not None:
        loss = loss + (rem * drem.to(compute_dtype)).sum()
    dq, dk, dv = torch.autograd.grad(loss, (qq, kk, vv))
    return o.detach(), rem.detach(), dq, dk, dv


def sb_attn_bwd_closed_form(q, k, v, do, drem, inv_temp=None, attend_current=False,
                            compute_dtype=torch.float64):
    """Gradients from the closed form the kernels implement (sb_varlen_bwd.py:416-430).

    g_ij = A_ij (dO_i.v_j - drem_i);  dz_ik = g_ik - beta_ik * sum_{j<=k} g_ij;
    dq = s dz K;  dk = s dz^T Q;  dv = A^T dO.   One dense problem, last dims [T, D].
    """
    if inv_temp is None:
        inv_temp = 1.0 / math.sqrt(q.shape[-1])
    cd = compute_dtype
    qd, kd, vd, dod = q.to(cd), k.to(cd), v.to(cd), do.to(cd)
    att, _ = _attention_matrix(qd, kd, inv_temp, attend_current, cd)
    T = q.shape[-2]
    mask = causal_mask(T, attend_current, device=q.device)
    beta = torch.sigmoid((qd @ kd.transpose(-1, -2)) * inv_temp).masked_fill(mask, 0.0)
    dA = dod @ vd.transpose(-1, -2) - drem.to(cd).unsqueeze(-1)
    g = att * dA
    dz = g - beta * g.cumsum(-1)
    dq = inv_temp * (dz @ kd)
    dk = inv_temp * (dz.transpose(-1, -2) @ qd)
    dv = att.transpose(-1, -2) @ dod
    return dq, dk, dv
