"""GPU parity: the HIP operator (through the C ABI) against the CPU oracle on identical
seeded inputs.  Tolerances are the ones the task states: forward o / rem max-abs
2e-2 (bf16) and 1e-4 (fp32); gradients 5e-2 relative L2 (bf16; fp32 is held to 2e-3).
float16 (tests/test_gpu_float16.py) is held to bf16's bounds divided by 8, the ratio of the unit roundoffs."""
import math
import os

import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, rel_l2, max_abs, cu_from_lengths, lognormal_lengths

pytestmark = pytest.mark.gpu

# float16: bf16's bounds times the ratio of the unit roundoffs (2^-11 against 2^-8)
FWD_TOL = {torch.bfloat16: 2e-2, torch.float32: 1e-4, torch.float16: 2.5e-3}
GRAD_TOL = {torch.bfloat16: 5e-2, torch.float32: 2e-3, torch.float16: 6.25e-3}


def _ops():
    from flame_amd import sb_attn, sb_attn_varlen
    return sb_attn, sb_attn_varlen


def _check_dense(B, H, T, D, dtype, attend_current=False, seed=0, in_scale=1.0, inv_temp=None,
                 with_drem=True, grads=True):
    sb_attn, _ = _ops()
    q, k, v = (randn((B, H, T, D), seed + i, in_scale, dtype) for i in range(3))
    do = randn((B, H, T, D), seed + 3, 1.0, dtype)
    drem = randn((B, H, T), seed + 4, 1.0, dtype) if with_drem else None
    print(f"dense B{B} H{H} T{T} D{D} {dtype} ac={attend_current} seed={seed}", flush=True)
    qg, kg, vg = (x.cuda().requires_grad_(grads) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg, inv_temp, attend_current=attend_current)
    assert o.dtype == dtype and rem.dtype == dtype and o.shape == (B, H, T, D) and rem.shape == (B, H, T)
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(
        q, k, v, do, drem, inv_temp=inv_temp, attend_current=attend_current, compute_dtype=torch.float32)
    assert max_abs(o.float().cpu(), o_ref) <= FWD_TOL[dtype]
    assert max_abs(rem.float().cpu(), rem_ref) <= FWD_TOL[dtype]
    if grads:
        loss = (o.float() * do.cuda().float()).sum()
        if with_drem:
            loss = loss + (rem.float() * drem.cuda().float()).sum()
        loss.backward()
        for name, g, ref in (("dq", qg.grad, dq_ref), ("dk", kg.grad, dk_ref), ("dv", vg.grad, dv_ref)):
            assert g.dtype == dtype and g.shape == ref.shape
            err = rel_l2(g.float().cpu(), ref)
            assert err <= GRAD_TOL[dtype], f"{name} rel-L2 {err}"


def test_config1_fp32_forward_and_grads():
    # benchmark configuration 1: B=2, H=4, T=512, d=64, fp32, N(0,1), scale 1/sqrt(64)
    _check_dense(2, 4, 512, 64, torch.float32, seed=0)


@pytest.mark.parametrize("T", [1, 2, 31, 64, 65, 130, 257])
@pytest.mark.parametrize("D", [8, 64, 96, 128])
def test_fp32_ragged_shapes(T, D):
    _check_dense(1, 2, T, D, torch.float32, seed=T + D)


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("T", [1, 33, 64, 127, 128, 129, 200, 512, 1000])
@pytest.mark.parametrize("D", [64, 128])
def test_bf16_dense(T, D, attend_current):
    _check_dense(2, 3, T, D, torch.bfloat16, attend_current=attend_current, seed=7 * T + D, in_scale=0.5)


def test_bf16_unit_variance_inputs_and_custom_temperature():
    _check_dense(1, 4, 384, 64, torch.bfloat16, seed=5, in_scale=1.0, inv_temp=0.2)


def test_bf16_other_head_dims_ride_the_matrix_core_kernels_zero_padded(monkeypatch):
    # padded to 64 / 128 on the host side; the padding is invisible in shapes and results
    _check_dense(1, 2, 150, 32, torch.bfloat16, seed=11, in_scale=0.5)
    _check_dense(1, 2, 150, 80, torch.bfloat16, seed=12, in_scale=0.5)
    _check_dense(2, 3, 300, 96, torch.bfloat16, attend_current=True, seed=14, in_scale=0.5)
    _check_varlen(3, 48, [70, 1, 200, 129], torch.bfloat16, seed=15)
    _check_varlen(2, 112, [300, 45], torch.bfloat16, attend_current=True, seed=16)
    # and the generic kernels at those head dims stay reachable
    monkeypatch.setenv("SBA_FORCE_GENERIC", "1")
    _check_dense(1, 2, 150, 80, torch.bfloat16, seed=12, in_scale=0.5)
    _check_varlen(3, 48, [70, 1, 200, 129], torch.bfloat16, seed=15)


def test_bf16_no_drem_and_no_grad():
    _check_dense(1, 2, 300, 64, torch.bfloat16, seed=21, in_scale=0.5, with_drem=False)
    _check_dense(1, 2, 300, 64, torch.bfloat16, seed=22, in_scale=0.5, grads=False)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_bf16_saturated_logits(D):
    # selected keys aligned with the queries so that |z| reaches 20 and more: exercises the
    # saturated sigmoid (the reference's softplus x>15 branch, softplus.py:9-10)
    sb_attn, _ = _ops()
    B, H, T = 1, 2, 320
    q = randn((B, H, T, D), 1, 0.5)
    k = randn((B, H, T, D), 2, 0.5)
    v = randn((B, H, T, D), 3, 1.0)
    qdir = q.mean(2, keepdim=True)
    qdir = qdir / qdir.norm(dim=-1, keepdim=True)
    g = torch.Generator().manual_seed(4)
    sel = torch.randperm(T, generator=g)[:12]
    k[:, :, sel] += 60.0 * qdir * torch.sign(torch.randn(12, generator=g))[None, None, :, None]
    q = q + 6.0 * qdir
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    z = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(D)
    assert z.abs().max() > 20
    do = randn((B, H, T, D), 5, 1.0, torch.bfloat16)
    print(f"saturated D{D} max|z|={float(z.abs().max()):.1f}", flush=True)
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(q, k, v, do, None, compute_dtype=torch.float64)
    assert torch.isfinite(o).all() and torch.isfinite(rem).all()
    assert max_abs(o.float().cpu(), o_ref) <= 2e-2 and max_abs(rem.float().cpu(), rem_ref) <= 2e-2
    (o.float() * do.cuda().float()).sum().backward()
    for g_, ref in ((qg.grad, dq_ref), (kg.grad, dk_ref), (vg.grad, dv_ref)):
        assert torch.isfinite(g_).all()
        assert rel_l2(g_.float().cpu(), ref) <= 5e-2


@pytest.mark.parametrize("D,rep", [(64, 1), (64, 100), (128, 1)])
def test_bf16_overflow_followed_by_exact_zero_inside_one_key_group(D, rep):
    # Inside the 32 keys that one lane chains over: logits of +80 (the running product of
    # 1 + e^z overflows) and, further left, logits of -200 (e^z is exactly 0 in fp32).  A chain
    # kept as that product meets inf * 0 there; the result must be finite and right: all
    # attention mass sits on the first +80 key, everything left of it gets weight 0.
    # rep = 100 repeats the batch row so that the large-grid forward kernel runs too.
    sb_attn, _ = _ops()
    H, T = 2, 300
    q, k, v = (randn((1, H, T, D), 140 + i, 0.5 if i < 2 else 1.0) for i in range(3))
    q[:, :, 200:, :] = 0
    q[:, :, 200:, 3] = 2.0 * math.sqrt(D)          # queries 200.. look along one coordinate
    k[:, :, 150:158, :] = 0
    k[:, :, 150:158, 3] = 40.0                     # logit +80
    k[:, :, 130:138, :] = 0
    k[:, :, 130:138, 3] = -100.0                   # logit -200
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    z = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(D)
    assert z.max() >= 79 and z.min() <= -199
    do = randn((1, H, T, D), 144, 1.0, torch.bfloat16)
    print(f"overflow-then-zero D{D} rep{rep}", flush=True)
    qg, kg, vg = (x.expand(rep, -1, -1, -1).contiguous().cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(q, k, v, do, None, compute_dtype=torch.float64)
    assert torch.isfinite(o).all() and torch.isfinite(rem).all()
    for b in (0, rep - 1):
        assert max_abs(o[b:b + 1].float().cpu(), o_ref) <= 2e-2 and max_abs(rem[b:b + 1].float().cpu(), rem_ref) <= 2e-2
    (o.float() * do.expand(rep, -1, -1, -1).cuda().float()).sum().backward()
    for g_, ref in ((qg.grad, dq_ref), (kg.grad, dk_ref), (vg.grad, dv_ref)):
        assert torch.isfinite(g_).all()
        assert rel_l2(g_[:1].float().cpu(), ref) <= 5e-2


def _check_varlen(H, D, lens, dtype, attend_current=False, seed=0, in_scale=0.5):
    _, sb_attn_varlen = _ops()
    N = sum(lens)
    cu = cu_from_lengths(lens)
    q, k, v = (randn((H, N, D), seed + i, in_scale, dtype) for i in range(3))
    do = randn((H, N, D), seed + 3, 1.0, dtype)
    drem = randn((H, N), seed + 4, 1.0, dtype)
    print(f"varlen H{H} D{D} docs={len(lens)} N={N} {dtype} ac={attend_current}", flush=True)
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn_varlen(qg, kg, vg, cu.cuda(), max(lens), attend_current=attend_current)
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(
        q, k, v, do, drem, attend_current=attend_current, cu_seqlens=cu.tolist(), compute_dtype=torch.float32)
    assert o.shape == (H, N, D) and rem.shape == (H, N)
    assert max_abs(o.float().cpu(), o_ref) <= FWD_TOL[dtype]
    assert max_abs(rem.float().cpu(), rem_ref) <= FWD_TOL[dtype]
    ((o.float() * do.cuda().float()).sum() + (rem.float() * drem.cuda().float()).sum()).backward()
    for name, g, ref in (("dq", qg.grad, dq_ref), ("dk", kg.grad, dk_ref), ("dv", vg.grad, dv_ref)):
        err = rel_l2(g.float().cpu(), ref)
        assert err <= GRAD_TOL[dtype], f"{name} rel-L2 {err}"


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_varlen_mixed_documents(dtype, attend_current):
    _check_varlen(4, 64, [1, 16, 129, 64, 300, 2, 128, 77], dtype, attend_current, seed=3)


def test_varlen_d128_and_single_document():
    _check_varlen(2, 128, [200, 31, 450], torch.bfloat16, seed=9)
    _check_varlen(2, 64, [333], torch.bfloat16, seed=10)


def test_varlen_lognormal_pack_8192():
    # config-3 style packing at a size the CPU oracle finishes in seconds
    lens = lognormal_lengths(8192, seed=0)
    _check_varlen(4, 64, lens, torch.bfloat16, seed=13)


def test_varlen_many_short_documents_stream_many_items_per_workgroup():
    # 2 x jobs x H = about 2500 (key block, head) items for the 256 resident dK/dV workgroups: ten
    # rounds each, most items a single step long (a finished dK/dV is staged and stored every
    # iteration), many second key blocks lying beyond the end of their document
    g = torch.Generator().manual_seed(21)
    lens = [int(x) for x in torch.randint(1, 201, (60,), generator=g)] + [64, 65, 128, 129, 256]
    _check_varlen(16, 64, lens, torch.bfloat16, seed=22)


def test_varlen_equals_dense_per_document():
    sb_attn, sb_attn_varlen = _ops()
    H, D, lens = 3, 64, [130, 64, 257]
    N = sum(lens)
    q, k, v = (randn((H, N, D), 40 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o, rem = sb_attn_varlen(q, k, v, cu_from_lengths(lens).cuda(), max(lens))
    s = 0
    for L in lens:
        od, rd = sb_attn(q[None, :, s:s + L], k[None, :, s:s + L], v[None, :, s:s + L])
        assert torch.equal(od[0], o[:, s:s + L]) and torch.equal(rd[0], rem[:, s:s + L])
        s += L


def test_strided_inputs_like_the_sba_layer():
    # q,k,v come from a [B, T, H*D] projection viewed as [B, H, T, D]; do is the gradient of a
    # 'b h l d -> b l (h d)' rearrange, i.e. strided (sba_layer.py:89-95)
    sb_attn, _ = _ops()
    B, H, T, D = 2, 4, 192, 64
    base = [randn((B, T, H * D), 50 + i, 0.5, torch.bfloat16).cuda().requires_grad_(True) for i in range(3)]
    q, k, v = (x.view(B, T, H, D).transpose(1, 2) for x in base)
    assert not q.is_contiguous()
    o, rem = sb_attn(q, k, v, None)
    w = randn((B, T, H * D), 53, 1.0, torch.bfloat16).cuda()
    (o.transpose(1, 2).reshape(B, T, H * D).float() * w.float()).sum().backward()
    qc, kc, vc = (x.detach().view(B, T, H, D).transpose(1, 2).contiguous().cpu() for x in base)
    do = w.view(B, T, H, D).transpose(1, 2).cpu()
    o_ref, rem_ref, dq_ref, dk_ref, dv_ref = O.sb_attn_grads_oracle(qc, kc, vc, do, None)
    assert max_abs(o.float().cpu(), o_ref) <= 2e-2
    for x, ref in zip(base, (dq_ref, dk_ref, dv_ref)):
        g = x.grad.view(B, T, H, D).transpose(1, 2)
        assert rel_l2(g.float().cpu(), ref) <= 5e-2


def test_mfma_and_generic_paths_agree():
    # two independent implementations of the same operator on the GPU
    sb_attn, _ = _ops()
    q, k, v = (randn((1, 4, 700, 64), 60 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o1, r1 = sb_attn(q, k, v)
    os.environ["SBA_FORCE_GENERIC"] = "1"
    try:
        o2, r2 = sb_attn(q, k, v)
    finally:
        del os.environ["SBA_FORCE_GENERIC"]
    assert max_abs(o1.float(), o2.float()) <= 2e-2 and max_abs(r1.float(), r2.float()) <= 1e-2


def test_forward_is_bitwise_repeatable():
    sb_attn, _ = _ops()
    q, k, v = (randn((2, 4, 513, 64), 70 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o1, r1 = sb_attn(q, k, v)
    o2, r2 = sb_attn(q, k, v)
    assert torch.equal(o1, o2) and torch.equal(r1, r2)


def test_row_mass_invariant_at_config2_size():
    # full size of benchmark configuration 2 (T=4096, H=16, d=64, bf16): size-independent properties
    # instead of the O(T^2)-memory oracle: with v = ones, o_i = sum_j A_ij = 1 - rem_i
    sb_attn, _ = _ops()
    B, H, T, D = 1, 16, 4096, 64
    q, k = (randn((B, H, T, D), 80 + i, 0.5, torch.bfloat16).cuda() for i in range(2))
    v = torch.ones(B, H, T, D, dtype=torch.bfloat16, device="cuda")
    o, rem = sb_attn(q, k, v)
    assert torch.isfinite(o).all()
    assert (o.float() + rem.float()[..., None] - 1).abs().max() <= 2e-2
    assert rem[:, :, 0].float().min() == 1 and o[:, :, 0].abs().max() == 0
    assert (rem.float() >= 0).all() and (rem.float() <= 1).all()
    # one head against the oracle
    o_ref, rem_ref = O.sb_attn_oracle(q[:, :1].cpu(), k[:, :1].cpu(), v[:, :1].cpu())
    assert max_abs(o[:, :1].float().cpu(), o_ref) <= 2e-2


def test_backward_is_bitwise_repeatable_and_matches_generic_path():
    # the MFMA backward has no atomics: two runs give identical bits; the generic kernels
    # (a second, independent implementation) agree within the gradient tolerance
    sb_attn, _ = _ops()
    q, k, v, do = (randn((1, 4, 600, 64), 90 + i, 0.5, torch.bfloat16).cuda() for i in range(4))
    drem = randn((1, 4, 600), 95, 1.0, torch.bfloat16).cuda()

    def grads():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn(qq, kk, vv)
        torch.autograd.backward([o, rem], [do, drem])
        return qq.grad, kk.grad, vv.grad

    g1, g2 = grads(), grads()
    assert all(torch.equal(a, b) for a, b in zip(g1, g2))
    os.environ["SBA_FORCE_GENERIC"] = "1"
    try:
        g3 = grads()
    finally:
        del os.environ["SBA_FORCE_GENERIC"]
    for a, b in zip(g1, g3):
        assert rel_l2(a.float(), b.float()) <= 2e-2


def test_sba_model_loss_matches_oracle_attention():
    # model wiring on the GPU: same weights, HIP operator (bf16 autocast) vs CPU oracle (fp32)
    from flame_amd.modeling_sba import SBAConfig, SBAForCausalLM
    cfg = SBAConfig(hidden_size=256, num_hidden_layers=2, num_heads=4, vocab_size=512)
    torch.manual_seed(0)
    ref = SBAForCausalLM(cfg)
    for layer in ref.model.layers:
        layer.attn.attn_fn = lambda q, k, v, t: O.sb_attn_oracle(q, k, v)
        layer.attn.attn_varlen_fn = lambda q, k, v, cu, ml: O.sb_attn_varlen_oracle(q, k, v, cu)
    gpu = SBAForCausalLM(cfg)
    gpu.load_state_dict(ref.state_dict())
    gpu.cuda()
    ids = torch.randint(0, 512, (1, 384))
    cu = torch.tensor([0, 100, 101, 300, 384], dtype=torch.int32)
    loss_ref, _ = ref(ids, labels=ids, cu_seqlens=cu)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        loss_gpu, _ = gpu(ids.cuda(), labels=ids.cuda(), cu_seqlens=cu.cuda(), max_seqlen=199)
        loss_dense, _ = gpu(ids.cuda(), labels=ids.cuda())
    loss_ref_dense, _ = ref(ids, labels=ids)
    assert abs(float(loss_gpu) - float(loss_ref)) <= 2e-2
    assert abs(float(loss_dense) - float(loss_ref_dense)) <= 2e-2
    loss_gpu.backward()
    assert all(torch.isfinite(p.grad).all() for p in gpu.parameters())


def test_sba_340m_width_train_step_runs():
    # config-5 style step at the 340M width (4 of the 24 layers to keep the test short):
    # packed varlen row, bf16 autocast, AdamW; loss finite and falling on a repeated batch
    from flame_amd.modeling_sba import SBAConfig, SBAForCausalLM
    from flame_amd.train_step import make_optimizer, train_step
    torch.manual_seed(0)
    model = SBAForCausalLM(SBAConfig(num_hidden_layers=4)).cuda()
    opt = make_optimizer(model, lr=1e-3)
    lens = lognormal_lengths(2048, seed=1)
    cu = cu_from_lengths(lens).cuda()
    ids = torch.randint(0, 32000, (1, 2048), device="cuda")
    losses = [float(train_step(model, opt, ids, ids, cu, max(lens))[0]) for _ in range(4)]
    print("losses", losses, flush=True)
    assert all(math.isfinite(x) for x in losses) and losses[-1] < losses[0]


def test_varlen_rejects_too_small_max_seqlens():
    _, sb_attn_varlen = _ops()
    q = randn((2, 300, 64), 1, 0.5, torch.bfloat16).cuda()
    with pytest.raises(ValueError, match="max_seqlens"):
        sb_attn_varlen(q, q, q, torch.tensor([0, 100, 300], dtype=torch.int32).cuda(), 150)


@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (96, torch.float16), (256, torch.bfloat16)])
def test_torch_compile_fullgraph_matches_eager(D, dtype):
    # the launchers are registered as stickbreaking_attention::{attn_fwd,attn_bwd,varlen_fwd,
    # varlen_bwd} custom ops (as the reference does, utils.py:20-39), so the op traces - also through the
    # zero-padding of a head dim and in float16
    sb_attn, sb_attn_varlen = _ops()
    assert hasattr(torch.ops.stickbreaking_attention, "attn_fwd")
    assert hasattr(torch.ops.stickbreaking_attention, "varlen_bwd")
    q, k, v, do = (randn((1, 2, 200, D), 100 + i, 0.5, dtype).cuda() for i in range(4))

    def f(q, k, v):
        o, rem = sb_attn(q, k, v)
        return o * 2, rem

    def run(fn):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, rem = fn(qq, kk, vv)
        torch.autograd.backward([o], [do])
        return o, rem, qq.grad, kk.grad, vv.grad

    eager = run(f)
    compiled = run(torch.compile(f, fullgraph=True))
    for a, b in zip(eager, compiled):
        assert torch.equal(a, b)


def test_small_and_large_grids_take_different_forward_kernels_and_agree(monkeypatch):
    # A launch whose longest sweep is long against the work of an average workgroup slot takes the segmented
    # forward (2, 3 or 4 key segments per sweep), one with many equal sweeps one workgroup per sweep.  Same rows
    # computed all ways (a batch of 1 vs the same sequence repeated 40 times).
    sb_attn, _ = _ops()
    q, k, v = (randn((1, 4, 1000, 64), 110 + i, 0.5, torch.bfloat16).cuda() for i in range(3))
    o1, r1 = sb_attn(q, k, v)                                   # 8 row-blocks x 4 heads = 32 workgroups
    for groups in ("2", "3"):
        monkeypatch.setenv("SBA_FWD_GROUPS", groups)
        og, rg = sb_attn(q, k, v)
        assert max_abs(o1.float(), og.float()) <= 2e-2 and max_abs(r1.float(), rg.float()) <= 1e-2
    monkeypatch.delenv("SBA_FWD_GROUPS")
    qq, kk, vv = (x.expand(40, -1, -1, -1).contiguous() for x in (q, k, v))
    o2, r2 = sb_attn(qq, kk, vv)                                # 1280 workgroups
    assert max_abs(o1.float(), o2[:1].float()) <= 2e-2 and max_abs(r1.float(), r2[:1].float()) <= 1e-2
    assert torch.equal(o2[0], o2[39]) and torch.equal(r2[0], r2[39])
    o_ref, rem_ref = O.sb_attn_oracle(q.cpu(), k.cpu(), v.cpu())
    assert max_abs(o2[39:].float().cpu(), o_ref) <= 2e-2 and max_abs(r2[39:].float().cpu(), rem_ref) <= 2e-2


@pytest.mark.parametrize("D", [64, 128])
def test_small_and_large_grids_take_different_backward_kernels_and_agree(D):
    # few workgroups with one dominating sweep: two-step-per-iteration dQ kernel (d = 64); many: one step per iteration.
    # Key-owner pass: the resident stream (d = 64) or the 64-key-block kernel (d = 128) on the
    # small grid, the kernel whose waves own their keys on the large one.
    sb_attn, _ = _ops()
    base = [randn((1, 4, 1000, D), 120 + i, 0.5, torch.bfloat16).cuda() for i in range(3)]
    do = randn((1, 4, 1000, D), 130, 1.0, torch.bfloat16).cuda()
    drem = randn((1, 4, 1000), 131, 1.0, torch.bfloat16).cuda()

    def grads(rep):
        q, k, v = (x.expand(rep, -1, -1, -1).contiguous().requires_grad_() for x in base)
        o, rem = sb_attn(q, k, v)
        torch.autograd.backward([o, rem], [do.expand(rep, -1, -1, -1).contiguous(), drem.expand(rep, -1, -1).contiguous()])
        return q.grad, k.grad, v.grad

    small, large = grads(1), grads(40)                      # 32 vs 1280 row-owner workgroups
    for a, b in zip(small, large):
        assert torch.equal(b[0], b[39])
        assert rel_l2(b[:1].float(), a.float()) <= 2e-2
    q, k, v = (x.cpu() for x in base)
    ref = O.sb_attn_grads_oracle(q, k, v, do.cpu(), drem.cpu())
    for a, b, r in zip(small, large, ref[-3:]):
        assert rel_l2(a.float().cpu(), r) <= 5e-2 and rel_l2(b[39:].float().cpu(), r) <= 5e-2


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("rep", [1, 40])
def test_gradient_of_rem_alone(D, rep):
    # dO = 0: everything comes from d_rem, which the matrix-core backward carries as the constant
    # d_rem * rem in its prefix tables (dz_ik = -beta_ik d_rem_i rem_i); dV must be exactly zero.
    # rep = 1 / 40: the small-grid and the large-grid kernels of both passes.
    sb_attn, _ = _ops()
    base = [randn((1, 4, 700, D), 140 + i, 0.5, torch.bfloat16).cuda() for i in range(3)]
    drem = randn((1, 4, 700), 143, 1.0, torch.bfloat16).cuda()
    q, k, v = (x.expand(rep, -1, -1, -1).contiguous().requires_grad_() for x in base)
    o, rem = sb_attn(q, k, v)
    torch.autograd.backward([o, rem], [torch.zeros_like(o), drem.expand(rep, -1, -1).contiguous()])
    assert torch.count_nonzero(v.grad) == 0
    qc, kc, vc = (x.cpu() for x in base)
    ref = O.sb_attn_grads_oracle(qc, kc, vc, torch.zeros_like(qc), drem.cpu())
    for g, r in zip((q.grad, k.grad), ref[-3:-1]):
        assert rel_l2(g[rep - 1:].float().cpu(), r) <= 5e-2
        assert torch.equal(g[0], g[rep - 1])


def _full_size_properties(fwd_bwd, v_shape_like, check_docs=None):
    """Size-independent properties of a forward+backward at a full benchmark size (no O(T^2)
    oracle needed): the backward is linear in the upstream gradients and bit-reproducible,
    and every result is finite."""
    do1, do2, dr1, dr2 = v_shape_like
    g1 = fwd_bwd(do1, dr1)
    g1b = fwd_bwd(do1, dr1)
    assert all(torch.equal(a, b) for a, b in zip(g1, g1b))          # no atomics: same bits
    g2 = fwd_bwd(do2, dr2)
    g12 = fwd_bwd((do1.float() + do2.float()).to(do1.dtype), (dr1.float() + dr2.float()).to(dr1.dtype))
    for a, b, c in zip(g1, g2, g12):
        assert torch.isfinite(c).all()
        # bf16 rounding of the summed upstream gradient and of each result: a few 2^-8 relative
        assert rel_l2(c.float(), a.float() + b.float()) <= 2e-2


def test_config3_size_packed_invariants():
    # full size of benchmark configuration 3: 65536 packed tokens, H=16, d=64, bf16, log-normal documents
    _, sb_attn_varlen = _ops()
    H, N, D = 16, 65536, 64
    lens = lognormal_lengths(N, seed=0)
    cu = cu_from_lengths(lens).cuda()
    q, k = (randn((H, N, D), 140 + i, 0.5, torch.bfloat16).cuda() for i in range(2))
    ones = torch.ones(H, N, D, dtype=torch.bfloat16, device="cuda")
    o, rem = sb_attn_varlen(q, k, ones, cu, max(lens))
    assert (o.float() + rem.float()[..., None] - 1).abs().max() <= 2e-2          # row mass
    starts = cu[:-1].long()
    assert rem[:, starts].float().min() == 1 and o[:, starts].abs().max() == 0   # first token of every document
    # block-diagonal: one document cut out and run alone gives the same rows (to a rounding step
    # of the bf16 outputs: alone, the document is a small launch and takes the segmented kernel,
    # which adds its partial sums in another order)
    d = max(range(len(lens)), key=lambda i: lens[i])
    a, b = int(cu[d]), int(cu[d + 1])
    o_d, rem_d = sb_attn_varlen(q[:, a:b].contiguous(), k[:, a:b].contiguous(), ones[:, a:b].contiguous(),
                                torch.tensor([0, b - a], dtype=torch.int32, device="cuda"), b - a)
    assert max_abs(o_d.float(), o[:, a:b].float()) <= 2 ** -7 and max_abs(rem_d.float(), rem[:, a:b].float()) <= 2 ** -7
    v = randn((H, N, D), 142, 0.5, torch.bfloat16).cuda()
    ups = [randn((H, N, D), 143 + i, 1.0, torch.bfloat16).cuda() for i in range(2)] + \
          [randn((H, N), 145 + i, 1.0, torch.bfloat16).cuda() for i in range(2)]

    def fwd_bwd(do, drem):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        oo, rr = sb_attn_varlen(qq, kk, vv, cu, max(lens))
        torch.autograd.backward([oo, rr], [do, drem])
        return qq.grad, kk.grad, vv.grad

    _full_size_properties(fwd_bwd, ups)


def test_config4_size_invariants():
    # full size of benchmark configuration 4: B=1, H=16, T=16384, d=128, bf16
    sb_attn, _ = _ops()
    B, H, T, D = 1, 16, 16384, 128
    q, k = (randn((B, H, T, D), 150 + i, 0.5, torch.bfloat16).cuda() for i in range(2))
    ones = torch.ones(B, H, T, D, dtype=torch.bfloat16, device="cuda")
    o, rem = sb_attn(q, k, ones)
    assert (o.float() + rem.float()[..., None] - 1).abs().max() <= 2e-2
    assert rem[:, :, 0].float().min() == 1 and o[:, :, 0].abs().max() == 0
    # causality: the first 1000 rows do not depend on what follows them
    o_p, rem_p = sb_attn(q[:, :, :1000].contiguous(), k[:, :, :1000].contiguous(), ones[:, :, :1000].contiguous())
    assert max_abs(o_p.float(), o[:, :, :1000].float()) <= 1e-2 and max_abs(rem_p.float(), rem[:, :, :1000].float()) <= 1e-2
    v = randn((B, H, T, D), 152, 1.0, torch.bfloat16).cuda()
    ups = [randn((B, H, T, D), 153 + i, 1.0, torch.bfloat16).cuda() for i in range(2)] + \
          [randn((B, H, T), 155 + i, 1.0, torch.bfloat16).cuda() for i in range(2)]

    def fwd_bwd(do, drem):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        oo, rr = sb_attn(qq, kk, vv)
        torch.autograd.backward([oo, rr], [do, drem])
        return qq.grad, kk.grad, vv.grad

    _full_size_properties(fwd_bwd, ups)


@pytest.mark.parametrize("dkv_kernel,D", [("", 64), ("own", 64), ("other", 64), ("stream8", 64), ("plain", 64),
                                          ("own", 128), ("other", 128), ("pair", 128)])
def test_randomized_packed_batches_mfma_vs_generic_backward(dkv_kernel, D, monkeypatch):
    # Seeded random packed batches (document counts, lengths around the 64/128 block edges,
    # head counts that are and are not multiples of 8, both masks): the MFMA kernels against the
    # generic vector-ALU kernels, an independent implementation, forward and all three gradients.
    # Every key-owner kernel is forced in turn (the library picks between them by grid size; the
    # stream with eight half-block producers and the plain 64-key-block kernel are selectable only).
    _, sb_attn_varlen = _ops()
    if dkv_kernel:
        monkeypatch.setenv("SBA_DKV_KERNEL", dkv_kernel)
    g = torch.Generator().manual_seed(1234)
    edges = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 384, 500, 777, 1025]
    for case in range(12):
        H = [1, 2, 3, 5, 8, 16][int(torch.randint(0, 6, (1,), generator=g))]
        n_docs = int(torch.randint(1, 40, (1,), generator=g))
        lens = [edges[int(torch.randint(0, len(edges), (1,), generator=g))] for _ in range(n_docs)]
        attend_current = bool(case % 2)
        N = sum(lens)
        cu = cu_from_lengths(lens).cuda()
        q, k, v, do = (randn((H, N, D), 1000 + 10 * case + i, 0.5 if i < 3 else 1.0, torch.bfloat16).cuda() for i in range(4))
        drem = randn((H, N), 1000 + 10 * case + 5, 1.0, torch.bfloat16).cuda()
        print(f"case {case}: D={D} dkv={dkv_kernel!r} H={H} docs={n_docs} N={N} attend_current={attend_current}", flush=True)

        def run():
            qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
            o, rem = sb_attn_varlen(qq, kk, vv, cu, max(lens), attend_current=attend_current)
            torch.autograd.backward([o, rem], [do, drem])
            return o, rem, qq.grad, kk.grad, vv.grad

        a = run()
        os.environ["SBA_FORCE_GENERIC"] = "1"
        try:
            b = run()
        finally:
            del os.environ["SBA_FORCE_GENERIC"]
        assert max_abs(a[0].float(), b[0].float()) <= 2e-2 and max_abs(a[1].float(), b[1].float()) <= 2e-2
        for x, y in zip(a[2:], b[2:]):
            assert torch.isfinite(x).all()
            assert rel_l2(x.float(), y.float()) <= 5e-2


@pytest.mark.parametrize("which", ["lean", "plain"])
def test_both_arrangements_of_the_one_step_dq_kernel_against_the_oracle(which, monkeypatch):
    # head_dim 64, grids above the two-step kernels' range: the library picks between the two arrangements of the
    # dQ kernel by launch size; each is forced here on a packed and a dense problem (ragged ends, both masks)
    # (576, 576 and 544 workgroups - 36, 36 and 17 row blocks times 16, 16 and 32 heads - none of which hangs on one
    # long sweep, so none takes the two-step kernel)
    monkeypatch.setenv("SBA_DQ_KERNEL", which)
    _check_varlen(16, 64, [300, 1, 129, 64, 517, 31, 1000, 128, 77, 640, 900], torch.bfloat16, False, seed=41)
    _check_varlen(16, 64, [2100, 65, 2300], torch.bfloat16, True, seed=42)
    _check_dense(4, 8, 2100, 64, torch.bfloat16, False, seed=43, in_scale=0.5)


def test_seeded_random_sweep_of_shapes_layouts_and_dtypes_against_the_oracle():
    # 120 seeded draws over what the fixed cases above leave between them: batch and head counts,
    # lengths from 1 to 2 000 at and off the 64 / 128 block edges, head dims on the matrix-core
    # kernels (64, 128) and on the zero-padded route (16, 32, 80, 96), both dtypes, both masks,
    # dense and packed (with empty documents), with and without a gradient for rem, inputs scaled
    # 0.5 and 0.75 (|o| stays below 4, where half a bf16 ulp of the output is 0.008).
    import random
    rng = random.Random(20240607)
    for case in range(120):
        D = rng.choice([64, 64, 128, 128, 16, 32, 80, 96])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.float32])
        ac = rng.random() < 0.3
        seed = rng.randrange(10 ** 6)
        scale = rng.choice([0.5, 0.75])
        if rng.random() < 0.5:
            B, H = rng.choice([1, 1, 2, 3]), rng.choice([1, 2, 3, 5])
            T = max(1, rng.choice([rng.randrange(1, 70), rng.randrange(1, 400), rng.randrange(1, 2000),
                                   128 * rng.randrange(1, 13), 64 * rng.randrange(1, 25) + rng.choice([-1, 0, 1])]))
            _check_dense(B, H, T, D, dtype, ac, seed=seed, in_scale=scale, with_drem=rng.random() < 0.8)
        else:
            H = rng.choice([1, 2, 4, 16])
            lens = [max(0 if rng.random() < 0.1 else 1,
                        rng.choice([rng.randrange(0, 40), rng.randrange(1, 300), rng.randrange(1, 1200),
                                    128 * rng.randrange(1, 6), 64 * rng.randrange(1, 10) + rng.choice([-1, 1])]))
                    for _ in range(rng.randrange(1, 14))]
            if sum(lens) == 0:
                lens.append(5)
            _check_varlen(H, D, lens, dtype, ac, seed=seed, in_scale=scale)


def test_forward_backward_captured_in_a_graph_replays_like_eager():
    # The C ABI allocates nothing and never synchronises, so a forward + backward can be captured
    # in a HIP graph.  Replayed three times with new input contents, with eager work in between,
    # every replay must give the bits of the eager run on the same inputs.
    sb_attn, _ = _ops()
    shape = (1, 4, 1024, 64)
    q, k, v = (randn(shape, 300 + i, 0.5, torch.bfloat16).cuda().requires_grad_(True) for i in range(3))
    do = randn(shape, 303, 1.0, torch.bfloat16).cuda()

    def step():
        o, rem = sb_attn(q, k, v)
        dq, dk, dv = torch.autograd.grad(o, (q, k, v), do)
        return o, rem, dq, dk, dv

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):            # warm-up on the capture stream, as torch asks
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(3):
        with torch.no_grad():
            for i, x in enumerate((q, k, v)):
                x.copy_(randn(shape, 310 + 10 * rep + i, 0.5, torch.bfloat16))
            do.copy_(randn(shape, 313 + 10 * rep, 1.0, torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()                        # eager, same inputs
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {rep}"


@pytest.mark.parametrize("D", [64, 128])
def test_recomputing_the_carries_in_the_backward_gives_the_same_bits(D, monkeypatch):
    # SBA_RECOMPUTE_CARRIES=1: the forward keeps no table and the backward repeats its sweep for the
    # carries alone.  Same kernels, same arithmetic: every result must be bit-identical.
    sb_attn, sb_attn_varlen = _ops()
    lens = [300, 1, 129, 700]
    cu = cu_from_lengths(lens).cuda()
    q, k, v, do = (randn((3, sum(lens), D), 400 + i, 0.5 if i < 3 else 1.0, torch.bfloat16).cuda() for i in range(4))
    drem = randn((3, sum(lens)), 405, 1.0, torch.bfloat16).cuda()

    def packed():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn_varlen(qq, kk, vv, cu, max(lens))
        torch.autograd.backward([o, rem], [do, drem])
        return o, rem, qq.grad, kk.grad, vv.grad

    def dense(rep):
        qq, kk, vv = (x[None].expand(rep, -1, -1, -1).contiguous().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn(qq, kk, vv, attend_current=True)
        torch.autograd.backward([o, rem], [do[None].expand(rep, -1, -1, -1).contiguous(), drem[None].expand(rep, -1, -1).contiguous()])
        return o, rem, qq.grad, kk.grad, vv.grad

    kept = [packed(), dense(1), dense(30)]              # small and large grids
    monkeypatch.setenv("SBA_RECOMPUTE_CARRIES", "1")
    again = [packed(), dense(1), dense(30)]
    for a, b in zip(kept, again):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.parametrize("D", [64, 128])
def test_fp32_runs_on_the_matrix_cores_bit_reproducibly_and_agrees_with_the_generic_kernels(D, monkeypatch):
    # fp32 takes the fp32 MFMA kernels (head_dim 64 and 128, no atomics): two runs give identical bits,
    # dense and packed; the generic vector-ALU kernels (a separate implementation) agree to fp32 accuracy
    sb_attn, sb_attn_varlen = _ops()
    q, k, v, do = (randn((2, 3, 333, D), 500 + i, 1.0 if i < 3 else 1.0).cuda() for i in range(4))
    drem = randn((2, 3, 333), 505).cuda()
    lens = [70, 1, 200, 129, 266]
    cu = cu_from_lengths(lens).cuda()
    qp, kp, vp, dop = (x.reshape(6, 333, D)[:, :, :].reshape(3, 666, D).contiguous() for x in (q, k, v, do))

    def dense():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn(qq, kk, vv)
        torch.autograd.backward([o, rem], [do, drem])
        return o, rem, qq.grad, kk.grad, vv.grad

    def packed():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (qp, kp, vp))
        o, rem = sb_attn_varlen(qq, kk, vv, cu, max(lens))
        torch.autograd.backward([o], [dop])
        return o, rem, qq.grad, kk.grad, vv.grad

    for fn in (dense, packed):
        a, b = fn(), fn()
        assert all(torch.equal(x, y) for x, y in zip(a, b))
        monkeypatch.setenv("SBA_FORCE_GENERIC", "1")
        c = fn()
        monkeypatch.delenv("SBA_FORCE_GENERIC")
        assert max_abs(a[0], c[0]) <= 1e-4 and max_abs(a[1], c[1]) <= 1e-4
        for x, y in zip(a[2:], c[2:]):
            assert rel_l2(x, y) <= 2e-3


def test_fp32_config1_in_memory_lean_mode(monkeypatch):
    # benchmark configuration 1 once more with the backward recomputing the carry table (fp32 MFMA kernels)
    monkeypatch.setenv("SBA_RECOMPUTE_CARRIES", "1")
    _check_dense(2, 4, 512, 64, torch.float32, seed=0)
