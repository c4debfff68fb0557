"""sba_bwd_static(), the backward that allocates nothing (its scratch is an array the library
holds on the GPU), against sba_bwd() with a caller-allocated scratch, through the C ABI.
Two calls in a row share the array, the second one smaller, so the second runs over the first
call's leftovers."""
import ctypes as C
import math

import pytest
import torch

from flame_amd import _lib
from helpers import randn, cu_from_lengths, rel_l2

pytestmark = pytest.mark.gpu


def _params(q, k, v, cu=None, max_len=None, sched=None):
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    if cu is None:
        B, H, T, D = q.shape
        p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
        desc = _lib.tensor4
    else:
        H, N, D = q.shape
        p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = cu.numel() - 1, H, max_len, N, D
        p.cu_seqlens, p.schedule, p.n_schedule = cu.data_ptr(), sched.data_ptr(), sched.shape[0]
        p.table_cols = _lib.table_columns(cu.cpu())
        desc = _lib.tensor3
    p.scale = 1.0 / math.sqrt(q.shape[-1])
    p.q, p.k, p.v = desc(q), desc(k), desc(v)
    p.stream = torch.cuda.current_stream().cuda_stream
    return p, desc


def _run_both(shape, dtype, seed, lens=None, keep_table=True):
    """Forward once, then the backward through both entry points; returns the two gradient triples."""
    lib = _lib.load()
    q, k, v, do = (randn(shape, seed + i, 0.5 if i < 3 else 1.0, dtype).cuda() for i in range(4))
    cu = sched = max_len = None
    if lens is not None:
        cu_host = cu_from_lengths(lens)
        cu, sched, max_len = cu_host.cuda(), _lib.build_schedule(cu_host, shape[0]).cuda(), max(lens)
    p, desc = _params(q, k, v, cu, max_len, sched)
    o = torch.empty_like(q)
    rem = torch.empty(q.shape[:-1], dtype=dtype, device="cuda")
    p.o = desc(o)
    p.rem = _lib.SbaVector(rem.data_ptr(), rem.stride(0) if cu is None else 0, rem.stride(-2) if cu is None else rem.stride(0))
    ws = torch.empty(max(int(lib.sba_workspace_bytes(C.byref(p))), 16), dtype=torch.uint8, device="cuda")
    if keep_table:
        p.save_for_backward = 1
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
    p.d_o = desc(do)
    need = int(lib.sba_bwd_scratch_bytes(C.byref(p)))
    assert need <= _lib.STATIC_SCRATCH_BYTES
    out = []
    for entry in (lib.sba_bwd, lib.sba_bwd_static):
        dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(3))
        p.dq, p.dk, p.dv = desc(dq), desc(dk), desc(dv)
        if entry is lib.sba_bwd:
            scratch = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
            p.bwd_scratch, p.bwd_scratch_bytes = scratch.data_ptr(), scratch.numel()
        else:
            p.bwd_scratch, p.bwd_scratch_bytes = None, 0      # ignored by the static entry point
        _lib.check(entry(C.byref(p)), entry.__name__)
        torch.cuda.synchronize()
        _lib.raise_if_gave_up(p, static_scratch_used=entry is lib.sba_bwd_static)      # the error word of this call
        out.append((dq, dk, dv))
    return out


def _same(a, b, exact):
    for x, y in zip(a, b):
        assert bool(torch.isfinite(x.float()).all())
        if exact:
            assert torch.equal(x, y)
        else:                      # the fp32 kernels add with atomics: equal to rounding only
            assert rel_l2(x.float().cpu(), y.float().cpu()) <= 2e-3


def test_static_backward_matches_sba_bwd_on_two_calls_in_a_row():
    print("static bwd: dense bf16 B1 H4 T1024 D64, then T300", flush=True)
    a, b = _run_both((1, 4, 1024, 64), torch.bfloat16, seed=0)
    _same(a, b, exact=True)
    a, b = _run_both((1, 4, 300, 64), torch.bfloat16, seed=10)          # smaller: runs over the leftovers
    _same(a, b, exact=True)


def test_static_backward_other_paths():
    print("static bwd: d128, recompute mode, packed, fp32, d256, float16", flush=True)
    a, b = _run_both((2, 2, 520, 128), torch.bfloat16, seed=20)
    _same(a, b, exact=True)
    a, b = _run_both((1, 2, 777, 64), torch.bfloat16, seed=30, keep_table=False)   # no table kept: the backward recomputes it
    _same(a, b, exact=True)
    a, b = _run_both((3, 900, 64), torch.bfloat16, seed=40, lens=[1, 130, 500, 64, 205])
    _same(a, b, exact=True)
    a, b = _run_both((1, 2, 200, 32), torch.float32, seed=50)
    _same(a, b, exact=False)
    a, b = _run_both((1, 2, 90, 64), torch.bfloat16, seed=60)
    _same(a, b, exact=True)
    a, b = _run_both((1, 2, 300, 256), torch.bfloat16, seed=70)         # head_dim 256
    _same(a, b, exact=True)
    a, b = _run_both((2, 2, 520, 64), torch.float16, seed=80)           # the float16 build of the kernels
    _same(a, b, exact=True)


def test_static_backward_refuses_what_does_not_fit():
    lib = _lib.load()
    q = torch.empty(1, 16, 16384, 128, dtype=torch.bfloat16, device="cuda")
    p, desc = _params(q, q, q)
    p.d_o = p.dq = p.dk = p.dv = desc(q)
    p.workspace, p.workspace_bytes = 1, 1 << 40      # never looked at: the size check comes first
    assert int(lib.sba_bwd_scratch_bytes(C.byref(p))) > _lib.STATIC_SCRATCH_BYTES
    assert lib.sba_bwd_static(C.byref(p)) == -8
    assert b"sba_bwd_static" in lib.sba_error_string(-8)
