"""The golden vectors under tests/golden (50-digit evaluation of the product formula and
central differences, see tests/golden/make_vectors.py) against the CPU oracle, the C brute
force, and -- on a GPU -- the HIP operator through the C ABI."""
import glob
import math
import os

import numpy as np
import pytest
import torch

from oracle import sb_oracle as O
from oracle import c_oracle
from helpers import max_abs, rel_l2, within

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "sb_*.npz")))
OUTPUTS = ("o", "rem", "dq", "dk", "dv")


# o / rem max-abs, gradients relative L2; float16: bf16's bounds times the ratio of the unit roundoffs (1/8)
_TOL = {torch.bfloat16: (2e-2, 5e-2), torch.float32: (1e-4, 2e-3), torch.float16: (2.5e-3, 6.25e-3)}
_NAME = {torch.bfloat16: "bf16", torch.float32: "fp32", torch.float16: "f16"}


def _load(path):
    z = np.load(path, allow_pickle=False)
    t = {n: torch.from_numpy(z[n]) for n in ("q", "k", "v", "do", "drem") + OUTPUTS}
    cu = torch.from_numpy(z["cu_seqlens"]) if "cu_seqlens" in z.files else None
    return t, cu, float(z["scale"]), bool(z["attend_current"])


def test_all_fixtures_present():
    assert len(GOLDEN) == 6


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_oracle_reproduces_golden_vectors(path):
    t, cu, scale, ac = _load(path)
    got = O.sb_attn_grads_oracle(t["q"], t["k"], t["v"], t["do"], t["drem"], inv_temp=scale, attend_current=ac,
                                 cu_seqlens=None if cu is None else cu.tolist(), compute_dtype=torch.float64)
    for name, g in zip(OUTPUTS, got):
        assert g.shape == t[name].shape
        assert max_abs(g, t[name]) <= 1e-12 * max(1.0, float(t[name].abs().max())), name


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_closed_form_gradients_reproduce_golden_vectors(path):
    # the gradient algebra the kernels implement, one (document, head) at a time
    t, cu, scale, ac = _load(path)
    packed = cu is not None
    bounds = cu.tolist() if packed else [0, t["q"].shape[-2]]
    heads = [(h,) for h in range(t["q"].shape[0])] if packed else \
        [(b, h) for b in range(t["q"].shape[0]) for h in range(t["q"].shape[1])]
    for idx in heads:
        for a, b in zip(bounds[:-1], bounds[1:]):
            x = {n: t[n][idx][a:b] for n in t}
            dq, dk, dv = O.sb_attn_bwd_closed_form(x["q"], x["k"], x["v"], x["do"], x["drem"], inv_temp=scale,
                                                   attend_current=ac)
            for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
                assert max_abs(g, x[name]) <= 1e-11 * max(1.0, float(x[name].abs().max())), (name, idx, a)
            o_c, rem_c, _ = c_oracle.forward(x["q"], x["k"], x["v"], scale, ac)
            assert max_abs(torch.from_numpy(o_c), x["o"]) <= 1e-12 and max_abs(torch.from_numpy(rem_c), x["rem"]) <= 1e-12
            gc = c_oracle.backward(x["q"], x["k"], x["v"], x["do"], x["drem"], scale, ac)
            for name, g in zip(("dq", "dk", "dv"), gc):
                assert max_abs(torch.from_numpy(g), x[name]) <= 1e-11 * max(1.0, float(x[name].abs().max())), ("c", name)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "f16"])
@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_hip_operator_reproduces_golden_vectors(path, dtype):
    from flame_amd import sb_attn, sb_attn_varlen
    t, cu, scale, ac = _load(path)
    print(f"golden {os.path.basename(path)} {dtype}", flush=True)
    fwd_tol, grad_tol = _TOL[dtype]   # inputs are bf16-exact (and with that float16-exact, down to values of 2^-15)
    q, k, v = (t[n].to(dtype).cuda().requires_grad_(True) for n in ("q", "k", "v"))
    if cu is None:
        o, rem = sb_attn(q, k, v, scale, attend_current=ac)
    else:
        lens = (cu[1:] - cu[:-1]).tolist()
        o, rem = sb_attn_varlen(q, k, v, cu.cuda(), max(lens), scale, attend_current=ac)
    loss = (o.float() * t["do"].float().cuda()).sum() + (rem.float() * t["drem"].float().cuda()).sum()
    loss.backward()
    label = f"golden {os.path.basename(path)} {_NAME[dtype]}"
    within(label, "o", max_abs(o.float().cpu(), t["o"]), fwd_tol)
    within(label, "rem", max_abs(rem.float().cpu(), t["rem"]), fwd_tol)
    for name, g in (("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        within(label, name, rel_l2(g.float().cpu(), t[name]), grad_tol)


# ---- matrix-core shapes: full forward, gradients along random directions ----
DIRECTIONAL = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "sbdir_*.npz")))


def _load_directional(path):
    z = np.load(path, allow_pickle=False)
    t = {n: torch.from_numpy(z[n]) for n in ("q", "k", "v", "do", "drem", "o", "rem", "directions", "slopes")}
    cu = torch.from_numpy(z["cu_seqlens"]) if "cu_seqlens" in z.files else None
    return t, cu, float(z["scale"]), bool(z["attend_current"])


def _slopes(grads, directions):
    # <gradient, direction> for the 3 inputs x n directions; one head, tokens x D
    return torch.stack([torch.stack([(g.double().reshape(u.shape) * u).sum() for u in directions[i]])
                        for i, g in enumerate(grads)])


def test_directional_fixtures_present():
    assert len(DIRECTIONAL) == 4


@pytest.mark.parametrize("path", DIRECTIONAL, ids=os.path.basename)
def test_oracle_reproduces_directional_vectors(path):
    t, cu, scale, ac = _load_directional(path)
    o, rem, dq, dk, dv = O.sb_attn_grads_oracle(t["q"], t["k"], t["v"], t["do"], t["drem"], inv_temp=scale,
                                                attend_current=ac, cu_seqlens=None if cu is None else cu.tolist(),
                                                compute_dtype=torch.float64)
    assert max_abs(o, t["o"]) <= 1e-12 and max_abs(rem, t["rem"]) <= 1e-12
    got = _slopes((dq, dk, dv), t["directions"])
    assert max_abs(got, t["slopes"]) <= 1e-10 * float(t["slopes"].abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "f16"])
@pytest.mark.parametrize("path", DIRECTIONAL, ids=os.path.basename)
def test_hip_operator_reproduces_directional_vectors(path, dtype):
    # D = 64 / 128 / 256: the matrix-core kernels (bf16, float16 and, up to 128, fp32 MFMA; fp32 at 256: generic)
    from flame_amd import sb_attn, sb_attn_varlen
    t, cu, scale, ac = _load_directional(path)
    print(f"golden {os.path.basename(path)} {dtype}", flush=True)
    fwd_tol, grad_tol = _TOL[dtype]
    q, k, v = (t[n].to(dtype).cuda().requires_grad_(True) for n in ("q", "k", "v"))
    if cu is None:
        o, rem = sb_attn(q, k, v, scale, attend_current=ac)
    else:
        lens = (cu[1:] - cu[:-1]).tolist()
        o, rem = sb_attn_varlen(q, k, v, cu.cuda(), max(lens), scale, attend_current=ac)
    loss = (o.float() * t["do"].float().cuda()).sum() + (rem.float() * t["drem"].float().cuda()).sum()
    loss.backward()
    label = f"golden {os.path.basename(path)} {_NAME[dtype]}"
    within(label, "o", max_abs(o.detach().float().cpu(), t["o"]), fwd_tol)
    within(label, "rem", max_abs(rem.detach().float().cpu(), t["rem"]), fwd_tol)
    grads = [g.detach().float().cpu() for g in (q.grad, k.grad, v.grad)]
    got = _slopes(grads, t["directions"])
    for i, name in enumerate(("dq", "dk", "dv")):
        for n, u in enumerate(t["directions"][i]):
            # An error e = g - g_true of size |e| <= tol |g| that is not aligned with the random
            # direction u shows as <e, u> ~ |e| |u| / sqrt(N); allow that much.  (A dropped term
            # or a wrong sign moves the slope by ~ |g| |u| / sqrt(N), far outside.)
            bound = grad_tol * float(grads[i].double().norm()) * float(u.norm()) / math.sqrt(u.numel())
            err = abs(float(got[i, n] - t["slopes"][i, n]))
            print(f"  {name}[{n}] slope {float(t['slopes'][i, n]):+.5f} error {err:.2e} bound {bound:.2e}", flush=True)
            within(label, name, err, bound)
