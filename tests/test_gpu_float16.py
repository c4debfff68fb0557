"""GPU parity of the float16 kernels (the bf16 matrix-core sources compiled for float16 elements; the
reference's kernels take whatever dtype the tensors have, sb_attn/sb_fwd.py:144-146) against the CPU
oracle on identical seeded inputs.  Tolerances: bf16's divided by 8, the ratio of the unit roundoffs
(2^-11 against 2^-8): o / rem max-abs 2.5e-3, gradients 6.25e-3 relative L2."""
import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, rel_l2, max_abs, cu_from_lengths, within
from test_gpu_parity import _check_dense, _check_varlen, _ops, FWD_TOL, GRAD_TOL

pytestmark = pytest.mark.gpu
F16 = torch.float16


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("T", [1, 33, 64, 127, 128, 129, 200, 512, 1000])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_float16_dense(T, D, attend_current):
    _check_dense(2, 3, T, D, F16, attend_current=attend_current, seed=7 * T + D + 1, in_scale=0.5)


def test_float16_other_head_dims_ride_the_matrix_core_kernels_zero_padded():
    _check_dense(1, 2, 150, 32, F16, seed=51, in_scale=0.5)
    _check_dense(2, 3, 300, 96, F16, attend_current=True, seed=52, in_scale=0.5)
    _check_dense(1, 2, 150, 200, F16, seed=53, in_scale=0.5)
    _check_varlen(3, 48, [70, 1, 200, 129], F16, seed=54)


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_float16_varlen(D, attend_current):
    _check_varlen(3, D, [300, 1, 129, 700, 64, 0, 5], F16, attend_current=attend_current, seed=55 + D)


def test_float16_unit_variance_inputs_no_drem_and_no_grad():
    _check_dense(1, 4, 384, 64, F16, seed=56, in_scale=1.0, inv_temp=0.2)
    _check_dense(1, 2, 300, 64, F16, seed=57, in_scale=0.5, with_drem=False)
    _check_dense(1, 2, 300, 128, F16, seed=58, in_scale=0.5, grads=False)


@pytest.mark.parametrize("D", [64, 128])
def test_float16_small_and_large_grids_take_different_kernels_and_agree(D):
    # one copy: the small-grid kernels (segmented forward, two-step dQ, dK/dV stream at head_dim 64); 40 copies: one sweep
    # per workgroup, register-lean dQ, own-keys / paired dK/dV.  Both against the oracle; all copies identical.
    sb_attn, _ = _ops()
    T = 1500
    base = [randn((1, 4, T, D), 60 + i, 0.5, F16) for i in range(3)]
    do, drem = randn((1, 4, T, D), 63, 1.0, F16), randn((1, 4, T), 64, 1.0, F16)
    ref = O.sb_attn_grads_oracle(*base, do, drem)
    for rep in (1, 40):
        print(f"float16 D{D} rep{rep}", flush=True)
        q, k, v = (x.cuda().expand(rep, -1, -1, -1).contiguous().requires_grad_() for x in base)
        o, rem = sb_attn(q, k, v)
        torch.autograd.backward([o, rem], [do.cuda().expand(rep, -1, -1, -1).contiguous(), drem.cuda().expand(rep, -1, -1).contiguous()])
        label = f"float16 d={D} T={T} x{rep}"
        within(label, "o", max_abs(o[:1].float().cpu(), ref[0]), FWD_TOL[F16])
        within(label, "rem", max_abs(rem[:1].float().cpu(), ref[1]), FWD_TOL[F16])
        for name, g, r in (("dq", q.grad, ref[2]), ("dk", k.grad, ref[3]), ("dv", v.grad, ref[4])):
            within(label, name, rel_l2(g[:1].float().cpu(), r), GRAD_TOL[F16])
            assert torch.equal(g[0], g[rep - 1])
        assert torch.equal(o[0], o[rep - 1])


def test_float16_lognormal_pack_and_recompute_mode_gives_the_same_bits(monkeypatch):
    from helpers import lognormal_lengths
    _, sb_attn_varlen = _ops()
    lens = lognormal_lengths(4096, seed=3)
    cu = cu_from_lengths(lens)
    H, D, N = 4, 64, sum(lens)
    q, k, v, do = (randn((H, N, D), 70 + i, 0.5 if i < 3 else 1.0, F16) for i in range(4))
    drem = randn((H, N), 75, 1.0, F16)

    def run():
        qq, kk, vv = (x.cuda().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn_varlen(qq, kk, vv, cu.cuda(), max(lens))
        torch.autograd.backward([o, rem], [do.cuda(), drem.cuda()])
        return o, rem, qq.grad, kk.grad, vv.grad

    kept = run()
    ref = O.sb_attn_grads_oracle(q, k, v, do, drem, cu_seqlens=cu.tolist())
    assert max_abs(kept[0].float().cpu(), ref[0]) <= FWD_TOL[F16] and max_abs(kept[1].float().cpu(), ref[1]) <= FWD_TOL[F16]
    for g, r in zip(kept[2:], ref[2:]):
        assert rel_l2(g.float().cpu(), r) <= GRAD_TOL[F16]
    monkeypatch.setenv("SBA_RECOMPUTE_CARRIES", "1")
    for x, y in zip(kept, run()):
        assert torch.equal(x, y)


def test_float16_saturated_logits_stay_finite_and_accurate():
    # |z| beyond 20 on selected keys (the reference's softplus x > 15 branch, softplus.py:9-10)
    import math
    sb_attn, _ = _ops()
    B, H, T, D = 1, 2, 320, 64
    q, k, v = randn((B, H, T, D), 81, 0.5), randn((B, H, T, D), 82, 0.5), randn((B, H, T, D), 83, 1.0)
    qdir = q.mean(2, keepdim=True)
    qdir = qdir / qdir.norm(dim=-1, keepdim=True)
    g = torch.Generator().manual_seed(84)
    sel = torch.randperm(T, generator=g)[:12]
    k[:, :, sel] += 60.0 * qdir * torch.sign(torch.randn(12, generator=g))[None, None, :, None]
    q = q + 6.0 * qdir
    q, k, v = (x.to(F16) for x in (q, k, v))
    z = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(D)
    assert z.abs().max() > 20
    do = randn((B, H, T, D), 85, 1.0, F16)
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    ref = O.sb_attn_grads_oracle(q, k, v, do, None, compute_dtype=torch.float64)
    (o.float() * do.cuda().float()).sum().backward()
    assert max_abs(o.float().cpu(), ref[0]) <= FWD_TOL[F16] and max_abs(rem.float().cpu(), ref[1]) <= FWD_TOL[F16]
    for g_, r in zip((qg.grad, kg.grad, vg.grad), ref[2:]):
        assert torch.isfinite(g_).all() and rel_l2(g_.float().cpu(), r) <= GRAD_TOL[F16]


def test_float16_on_the_generic_kernels(monkeypatch):
    # the vector-ALU kernels in float16 storage (fp32 arithmetic): forced for everything, and for the backward alone
    monkeypatch.setenv("SBA_FORCE_GENERIC", "1")
    _check_dense(1, 2, 200, 64, F16, seed=90, in_scale=0.5)
    _check_dense(1, 2, 130, 200, F16, attend_current=True, seed=92, in_scale=0.5)
    _check_varlen(2, 80, [130, 45], F16, seed=91)
    monkeypatch.delenv("SBA_FORCE_GENERIC")
    monkeypatch.setenv("SBA_FORCE_GENERIC_BWD", "1")
    _check_dense(1, 2, 300, 128, F16, seed=93, in_scale=0.5)
