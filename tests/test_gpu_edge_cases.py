"""GPU edge cases of the operator: empty inputs, one-token sequences, zero-length documents inside a
packed batch, and the longest row a flame data loader produces (65536 tokens, dense)."""
import pytest
import torch

from oracle import sb_oracle as O
from helpers import randn, rel_l2, max_abs, cu_from_lengths

pytestmark = pytest.mark.gpu


def test_empty_inputs_launch_nothing_and_keep_the_graph():
    from flame_amd import sb_attn, sb_attn_varlen
    q = torch.zeros(2, 4, 0, 64, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    o, rem = sb_attn(q, q, q)
    assert o.shape == (2, 4, 0, 64) and rem.shape == (2, 4, 0)
    (o.float().sum() + rem.float().sum()).backward()
    assert q.grad.shape == q.shape
    qv = torch.zeros(4, 0, 64, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    o, rem = sb_attn_varlen(qv, qv, qv, torch.zeros(1, dtype=torch.int32), 0)
    assert o.shape == (4, 0, 64) and rem.shape == (4, 0)
    (o.float().sum() + rem.float().sum()).backward()
    assert qv.grad.shape == qv.shape


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_one_and_two_token_sequences(dtype, attend_current):
    # strict mode: the first token sees no key (o = 0, rem = 1, no gradient)
    from flame_amd import sb_attn
    for T in (1, 2):
        q, k, v, do = (randn((2, 3, T, 64), 700 + i, 0.5 if i < 3 else 1.0, dtype) for i in range(4))
        drem = randn((2, 3, T), 705, 1.0, dtype)
        print(f"T={T} {dtype} attend_current={attend_current}", flush=True)
        qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
        o, rem = sb_attn(qg, kg, vg, attend_current=attend_current)
        torch.autograd.backward([o, rem], [do.cuda(), drem.cuda()])
        o_ref, rem_ref, dq, dk, dv = O.sb_attn_grads_oracle(q, k, v, do, drem, attend_current=attend_current)
        tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
        assert max_abs(o.detach().float().cpu(), o_ref) <= tol and max_abs(rem.detach().float().cpu(), rem_ref) <= tol
        if not attend_current:
            assert torch.equal(o[:, :, 0].float().cpu(), torch.zeros(2, 3, 64)) and torch.equal(rem[:, :, 0].float().cpu(), torch.ones(2, 3))
        for got, ref in ((qg.grad, dq), (kg.grad, dk), (vg.grad, dv)):
            assert torch.isfinite(got).all()
            assert max_abs(got.float().cpu(), ref) <= (5e-2 if dtype == torch.bfloat16 else 2e-3) * max(1.0, float(ref.abs().max()))


def test_zero_length_documents_inside_a_pack():
    # consecutive equal entries of cu_seqlens are documents without tokens: they take no part
    from flame_amd import sb_attn_varlen
    lens = [0, 70, 0, 0, 1, 200, 0, 129, 0]
    cu = cu_from_lengths(lens)
    N = sum(lens)
    q, k, v, do = (randn((3, N, 64), 710 + i, 0.5 if i < 3 else 1.0, torch.bfloat16) for i in range(4))
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn_varlen(qg, kg, vg, cu.cuda(), max(lens))
    torch.autograd.backward([o], [do.cuda()])
    o_ref, rem_ref, dq, dk, dv = O.sb_attn_grads_oracle(q, k, v, do, None, cu_seqlens=[c for c in cu.tolist()])
    assert max_abs(o.detach().float().cpu(), o_ref) <= 2e-2 and max_abs(rem.detach().float().cpu(), rem_ref) <= 2e-2
    for got, ref in ((qg.grad, dq), (kg.grad, dk), (vg.grad, dv)):
        assert rel_l2(got.float().cpu(), ref) <= 5e-2
    # the same pack without the empty documents gives the same bits
    cu2 = cu_from_lengths([L for L in lens if L])
    o2, rem2 = sb_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu2.cuda(), max(lens))
    assert torch.equal(o2, o.detach()) and torch.equal(rem2, rem.detach())


def test_longest_dense_row_65536_tokens_invariants():
    # the longest row a data loader hands over (one document of 65536 tokens): mass conservation with
    # v = 1, the first rows against the oracle on a prefix (causality), finite gradients, and the carry
    # tables' 64-bit indexing (262 656 table columns per head)
    from flame_amd import sb_attn
    T, H, D = 65536, 2, 64
    q, k = (randn((1, H, T, D), 720 + i, 0.5, torch.bfloat16).cuda() for i in range(2))
    v = torch.ones(1, H, T, D, dtype=torch.bfloat16, device="cuda")
    qg, kg, vg = (x.requires_grad_(True) for x in (q, k, v))
    print("dense T=65536 forward + backward", flush=True)
    o, rem = sb_attn(qg, kg, vg)
    assert float((o.detach().float()[..., 0] + rem.detach().float() - 1).abs().max()) <= 2e-2
    do = randn((1, H, T, D), 723, 1.0, torch.bfloat16).cuda()
    torch.autograd.backward([o], [do])
    for g in (qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(g).all()
    P = 1024
    o_ref, rem_ref = O.sb_attn_oracle(q[:, :, :P].float().cpu(), k[:, :, :P].float().cpu(), v[:, :, :P].float().cpu())
    assert max_abs(o.detach()[:, :, :P].float().cpu(), o_ref) <= 2e-2 and max_abs(rem.detach()[:, :, :P].float().cpu(), rem_ref) <= 2e-2
    # the last rows against the oracle on the keys they can still feel (weights beyond ~200 keys are below 2^-126
    # for these inputs: beta is about one half)
    W = 2048
    qs, ks, vs = (x[:, :1, T - W:].float().cpu() for x in (q, k, v))
    o_tail, rem_tail = O.sb_attn_oracle(qs, ks, vs)
    assert max_abs(o.detach()[:, :1, T - 256:].float().cpu(), o_tail[:, :, W - 256:]) <= 2e-2


@pytest.mark.parametrize("D", [64, 128, 256])
def test_carries_that_underflow_to_zero(D):
    # Logits around +6 in natural units (beta ~ 0.998): the product of (1 - beta) entering a key block is
    # below the fp32 range after a few tens of keys, so the carry tables hold exact zeros for almost every
    # (query, key block) pair, and the backward's chains start from a zero carry (an infinite W, NaNs mapped
    # to 0 by the clamps).  Everything must stay finite and agree with the oracle: only the nearest keys
    # have weight, all gradients of far keys are exactly zero.
    from flame_amd import sb_attn
    B, H, T = 1, 2, 1024
    g = torch.Generator().manual_seed(900 + D)
    base = torch.randn(D, generator=g)
    base = base / base.norm()
    amp = (6.0 * D ** 0.5) ** 0.5                      # q . k / sqrt(D) ~ 6
    q = (amp * base + 0.05 * torch.randn(B, H, T, D, generator=g)).to(torch.bfloat16)
    k = (amp * base + 0.05 * torch.randn(B, H, T, D, generator=g)).to(torch.bfloat16)
    v = randn((B, H, T, D), 903, 0.25, torch.bfloat16)     # |o| <= 1: the tolerance on o is an absolute one
    do = randn((B, H, T, D), 904, 1.0, torch.bfloat16)
    drem = randn((B, H, T), 905, 1.0, torch.bfloat16)
    print(f"underflowing carries, D={D}", flush=True)
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    torch.autograd.backward([o, rem], [do.cuda(), drem.cuda()])
    o_ref, rem_ref, dq, dk, dv = O.sb_attn_grads_oracle(q, k, v, do, drem, compute_dtype=torch.float64)
    for t in (o, rem, qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(t).all()
    assert max_abs(o.detach().float().cpu(), o_ref.float()) <= 2e-2
    assert max_abs(rem.detach().float().cpu(), rem_ref.float()) <= 2e-2
    for got, ref in ((qg.grad, dq), (kg.grad, dk), (vg.grad, dv)):
        assert rel_l2(got.float().cpu(), ref.float()) <= 5e-2


def test_error_word_set_from_the_host_is_reported_and_cleared_by_the_next_backward():
    # The error word of the bf16 matrix-core backward (last 256 bytes of its scratch) is cleared by the
    # dQ pass and may be set by the stream kernel.  No kernel is made to give up here: the host writes the
    # word between the two passes of a backward issued as two calls (SbaParams.bwd_phases), which is what a
    # wave abandoning its wait in the second pass would have done.  sba_bwd_gave_up must report it, the
    # Python check must raise, and a complete backward on the same scratch must clear it again.
    import ctypes as C
    import math
    from flame_amd import _lib
    lib = _lib.load()
    B, H, T, D = 1, 2, 512, 64
    q, k, v, do = (randn((B, H, T, D), 760 + i, 0.5 if i < 3 else 1.0, torch.bfloat16).cuda() for i in range(4))
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.SBA_DTYPE_BF16
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
    p.scale = 1.0 / math.sqrt(D)
    p.q, p.k, p.v = _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v)
    p.stream = torch.cuda.current_stream().cuda_stream
    o, rem = torch.empty_like(q), torch.empty(B, H, T, dtype=q.dtype, device="cuda")
    p.o, p.rem = _lib.tensor4(o), _lib.SbaVector(rem.data_ptr(), rem.stride(0), rem.stride(1))
    ws = torch.empty(int(lib.sba_workspace_bytes(C.byref(p))), dtype=torch.uint8, device="cuda")
    p.save_for_backward, p.workspace, p.workspace_bytes = 1, ws.data_ptr(), ws.numel()
    _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
    dq, dk, dv = (torch.empty_like(q) for _ in range(3))
    p.d_o, p.dq, p.dk, p.dv = _lib.tensor4(do), _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv)
    scratch = torch.empty(int(lib.sba_bwd_scratch_bytes(C.byref(p))), dtype=torch.uint8, device="cuda")
    p.bwd_scratch, p.bwd_scratch_bytes = scratch.data_ptr(), scratch.numel()
    word = scratch[-256:-252].view(torch.int32)
    flag = C.c_int(-1)
    print("error word: two-call backward with the word written by the host in between", flush=True)
    p.bwd_phases = 1
    _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd pass 1")
    torch.cuda.synchronize()
    assert int(word.item()) == 0                                   # cleared by the dQ pass
    word.fill_(1)
    p.bwd_phases = 2
    _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd pass 2")          # runs normally and leaves the word alone
    assert lib.sba_bwd_gave_up(C.byref(p), 0, C.byref(flag)) == 0 and flag.value == 1
    with pytest.raises(RuntimeError, match="abandoned a bounded internal wait"):
        _lib.raise_if_gave_up(p)
    first = (dq.clone(), dk.clone(), dv.clone())
    p.bwd_phases = 0
    _lib.check(lib.sba_bwd(C.byref(p)), "sba_bwd")
    assert lib.sba_bwd_gave_up(C.byref(p), 0, C.byref(flag)) == 0 and flag.value == 0
    _lib.raise_if_gave_up(p)
    for a, b in zip(first, (dq, dk, dv)):                          # the word changes nothing in the results
        assert torch.equal(a, b)
