"""Packed (varlen) stick-breaking attention, [H, sumT, D] + cu_seqlens.

Host-side mirror of custom_models/sba/stickbreaking_attention/sb_varlen/__init__.py:24-82.
The reference's 3-D launch grid with long/short head pairing
(sb_varlen_fwd.py:288-289, 472-475) is replaced by a row-block schedule built once per
cu_seqlens on the host (sba_build_schedule) and reused by every layer that sees the same
packing.
"""
from __future__ import annotations

import ctypes as C
import math
import weakref
from typing import Optional

import torch

from .. import _lib
from . import profiling
from .utils import custom_op

# Schedules are cached per cu_seqlens TENSOR OBJECT (identity + version counter), so the 24
# layers of a model that receive the same tensor share one host sync; a data_ptr-based key
# would be unsafe because the caching allocator reuses addresses.
_SCHEDULES: dict = {}


def _schedule_for(cu_seqlens: torch.Tensor, n_heads: int, device: torch.device):
    """(cu int32 on `device` with leading 0, schedule on `device`, n_jobs, max_len, total, table
    columns).  `cu_seqlens` itself may live anywhere (a CPU tensor spares the host sync); what the
    kernels read is placed on the device of q.  The job order depends on the launch size
    (jobs x heads): one entry per cu_seqlens tensor, device and order."""
    key = (id(cu_seqlens), device)
    hit = _SCHEDULES.get(key)
    if hit is not None and hit[0]() is cu_seqlens and hit[1] == cu_seqlens._version:
        entry = hit[2]
        if (entry[2] * n_heads >= _lib.DOC_MAJOR_GRID) == hit[3]:
            return entry
    cu_host = cu_seqlens.detach().to("cpu", torch.int32)   # one host sync per new packing
    if cu_host.dim() != 1 or cu_host.numel() < 2 or int(cu_host[0]) != 0:
        raise ValueError("cu_seqlens must be 1-D, start with 0 and hold at least one document")
    lens = cu_host[1:] - cu_host[:-1]
    if bool((lens < 0).any()):
        raise ValueError("cu_seqlens must be non-decreasing")
    sched = _lib.build_schedule(cu_host, n_heads)
    entry = (cu_host.to(device), sched.to(device), sched.shape[0], int(lens.max()), int(cu_host[-1]),
             _lib.table_columns(cu_host))
    ref = weakref.ref(cu_seqlens, lambda _r, key=key: _SCHEDULES.pop(key, None))
    _SCHEDULES[key] = (ref, cu_seqlens._version, entry, sched.shape[0] * n_heads >= _lib.DOC_MAJOR_GRID)
    return entry


def _params(q, k, v, n_docs, max_seqlens, inv_temp, attend_current):
    H, N, D = q.shape
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = n_docs, H, max_seqlens, N, D
    p.attend_current = int(bool(attend_current))
    p.scale = float(inv_temp)
    p.q, p.k, p.v = _lib.tensor3(q), _lib.tensor3(k), _lib.tensor3(v)
    p.stream = _lib.current_stream_handle(q.device)
    return p


def _bind_schedule(p, q, cu_seqlens, max_seqlens):
    cu_dev, sched, n_jobs, max_len, total, cols = _schedule_for(cu_seqlens, q.shape[0], q.device)
    if total != q.shape[1]:
        raise ValueError(f"cu_seqlens ends at {total} but q has {q.shape[1]} tokens")
    if max_len > max_seqlens:
        raise ValueError(f"max_seqlens={max_seqlens} is smaller than the longest document ({max_len})")
    p.cu_seqlens, p.schedule, p.n_schedule, p.table_cols = cu_dev.data_ptr(), sched.data_ptr(), n_jobs, cols
    # the library chooses its kernels from the longest sweep of the launch: give it the real longest document,
    # which max_seqlens may only bound
    p.seq_len = max(max_len, 1)
    return n_jobs


def _columns(q, cu_seqlens, max_seqlens: int) -> int:
    """Carry-table columns of this packing: exact from the cached schedule, or, while
    torch.compile traces (no look at cu_seqlens' values), a bound from the shapes."""
    if torch.compiler.is_compiling():
        return _lib.packed_columns_bound(q.shape[1], cu_seqlens.numel() - 1, max_seqlens)
    return _schedule_for(cu_seqlens, q.shape[0], q.device)[5]


def workspace_bytes(q, cu_seqlens, max_seqlens: int) -> int:
    """What lives from the forward to the backward (the forward's carry table): one float per
    query and visible 64-key block of its own document, sized from the actual document lengths."""
    cols = _columns(q, cu_seqlens, max_seqlens)
    if torch.compiler.is_compiling():
        return _lib.workspace_upper_bound(q.shape[0], cols)
    p = _params(q, q, q, 1, max_seqlens, 1.0, False)
    p.cu_seqlens, p.table_cols = 1, cols          # only "packed or not" and the size matter here
    return int(_lib.load().sba_workspace_bytes(C.byref(p)))


def bwd_scratch_bytes(q, cu_seqlens, max_seqlens: int, have_workspace=True) -> int:
    """What the backward needs for the duration of its call only (one table more when the forward
    kept none)."""
    cols = _columns(q, cu_seqlens, max_seqlens)
    if torch.compiler.is_compiling():
        H, N, D = q.shape
        return _lib.bwd_scratch_upper_bound(H, cols, N, D)
    p = _params(q, q, q, 1, max_seqlens, 1.0, False)
    p.cu_seqlens, p.table_cols = 1, cols
    p.workspace = 1 if have_workspace else None       # only NULL or not is looked at
    return int(_lib.load().sba_bwd_scratch_bytes(C.byref(p)))


# Registered names as in the reference (sb_varlen_fwd.py:449, sb_varlen_bwd.py:523).
@custom_op("varlen_fwd", mutates_args=("o", "rem", "ws"))
def _compileable_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                         max_seqlens: int, logit_scale: float, attend_current: bool, save: bool,
                         o: torch.Tensor, rem: torch.Tensor, ws: torch.Tensor) -> None:
    lib = _lib.load()
    p = _params(q, k, v, cu_seqlens.numel() - 1, max_seqlens, logit_scale, attend_current)
    if _bind_schedule(p, q, cu_seqlens, max_seqlens) == 0:
        return
    p.o = _lib.tensor3(o)
    p.rem = _lib.SbaVector(rem.data_ptr(), 0, rem.stride(0))
    p.save_for_backward = int(save)
    if save:
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    profiling.mark("start")
    _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
    profiling.mark("fwd")


@custom_op("varlen_bwd", mutates_args=("dq", "dk", "dv", "scratch"))
def _compileable_backward(do: torch.Tensor, dr: Optional[torch.Tensor], q: torch.Tensor, k: torch.Tensor,
                          v: torch.Tensor, cu_seqlens: torch.Tensor, max_seqlens: int, ws: torch.Tensor,
                          scratch: torch.Tensor, logit_scale: float, attend_current: bool, dq: torch.Tensor,
                          dk: torch.Tensor, dv: torch.Tensor) -> None:
    lib = _lib.load()
    p = _params(q, k, v, cu_seqlens.numel() - 1, max_seqlens, logit_scale, attend_current)
    if _bind_schedule(p, q, cu_seqlens, max_seqlens) == 0:
        return
    p.d_o = _lib.tensor3(do)
    if dr is not None:
        p.d_rem = _lib.SbaVector(dr.data_ptr(), 0, dr.stride(0))
    p.dq, p.dk, p.dv = _lib.tensor3(dq), _lib.tensor3(dk), _lib.tensor3(dv)
    if ws.numel() > 16:                   # a 16-byte stand-in means: nothing was kept, recompute the carries
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    p.bwd_scratch, p.bwd_scratch_bytes = scratch.data_ptr(), scratch.numel()
    profiling.launch_bwd(lib, p)


def attention_weights_varlen(q, k, cu_seqlens, max_seqlens, inv_temp=None, attend_current=False):
    """The attention weights of a packed batch as float32 [H, sum T, sum T], every document's block on the diagonal,
    zero elsewhere: what the reference's `varlen_fwd` returns as `W` under `return_attention=True`
    (sb_varlen_fwd.py:409-446).  For inspection and tests: a vector-ALU kernel, (sum T)^2 floats per head."""
    if not q.is_cuda:
        raise RuntimeError("stick-breaking attention runs on the GPU only (HIP kernels); there is no CPU path")
    if q.shape != k.shape or q.dim() != 3 or q.dtype != k.dtype:
        raise ValueError("q, k must both be [H, sum T, D] of one dtype")
    _lib.check_supported(q)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    H, N, _ = q.shape
    W = torch.zeros((H, N, N), dtype=torch.float32, device=q.device)
    if W.numel():
        q, k = _lib.usable(q.detach()), _lib.usable(k.detach())
        p = _params(q, k, k, cu_seqlens.numel() - 1, max_seqlens, inv_temp, attend_current)
        if _bind_schedule(p, q, cu_seqlens, max_seqlens) != 0:
            _lib.check(_lib.load().sba_attention_weights(C.byref(p), W.data_ptr()), "sba_attention_weights")
    return W


def varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current=False, no_grad=False,
               return_attention=False):
    if return_attention:                 # the reference's debug output rides along as a fourth result
        return (*varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current, no_grad),
                attention_weights_varlen(q, k, cu_seqlens, max_seqlens, logit_scale, attend_current))
    o = torch.empty_like(q)
    rem = torch.empty(q.shape[:-1], dtype=q.dtype, device=q.device)
    # above the workspace budget nothing is kept and the backward recomputes the carries (_lib.recompute_carries)
    nbytes = 16 if no_grad else max(workspace_bytes(q, cu_seqlens, max_seqlens), 16)
    keep = not (no_grad or _lib.recompute_carries(nbytes))
    if not keep:
        nbytes = 16
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    _compileable_forward(q, k, v, cu_seqlens, int(max_seqlens), float(logit_scale), bool(attend_current),
                         keep, o, rem, ws)
    return o, rem, ws


def varlen_bwd(do, dr, q, k, v, cu_seqlens, max_seqlens, ws, logit_scale, attend_current=False):
    dq, dk, dv = _lib.empty_grads_like(q, k, v)     # one allocation when q, k, v are slices of one tensor
    # freed when this call returns: only the forward's table is kept between the two directions
    scratch = torch.empty(max(bwd_scratch_bytes(q, cu_seqlens, max_seqlens, ws.numel() > 16), 16), dtype=torch.uint8,
                          device=q.device)
    _compileable_backward(do, dr, q, k, v, cu_seqlens, int(max_seqlens), ws, scratch, float(logit_scale),
                          bool(attend_current), dq, dk, dv)
    return dq, dk, dv


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        if not q.is_cuda:
            raise RuntimeError("stick-breaking attention runs on the GPU only (HIP kernels); "
                               "there is no CPU path")
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
        if not (q.device == k.device == v.device):
            raise ValueError("q, k, v must be on the same device")
        if not (q.shape == k.shape == v.shape) or q.dim() != 3:
            raise ValueError("q, k, v must all be [H, total_tokens, D]")
        _lib.check_supported(q)
        no_grad = not any(ctx.needs_input_grad[:3])
        ctx.head_dim = q.shape[-1]
        Dp = _lib.matrix_core_head_dim(q)
        q, k, v = (_lib.usable(_lib.pad_head_dim(x, Dp)) for x in (q, k, v))
        o, rem, ws = varlen_fwd(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, no_grad)
        ctx.save_for_backward(q, k, v, ws, cu_seqlens)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_seqlens
        ctx.attend_current = attend_current
        ctx.set_materialize_grads(False)
        return _lib.cut_head_dim(o, ctx.head_dim), rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, ws, cu_seqlens = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(q)
        do = _lib.usable(_lib.pad_head_dim(do, q.shape[-1]))
        if drem is not None:
            drem = drem.contiguous()
        dq, dk, dv = varlen_bwd(do, drem, q, k, v, cu_seqlens, ctx.max_seqlens, ws, ctx.logit_scale,
                                ctx.attend_current)
        return (*(_lib.cut_head_dim(g, ctx.head_dim) for g in (dq, dk, dv)), None, None, None, None)


# cu_seqlens without its leading 0 (the reference's inner convention) -> the tensor with the 0 in front, one per
# source tensor and version, so that the 24 layers of a model that pass the same tensor share one schedule entry.
_WITH_ZERO: dict = {}


def _with_leading_zero(cu_seqlens: torch.Tensor) -> torch.Tensor:
    if torch.compiler.is_compiling():
        return torch.cat([cu_seqlens.new_zeros(1), cu_seqlens])
    key = id(cu_seqlens)
    hit = _WITH_ZERO.get(key)
    if hit is not None and hit[0]() is cu_seqlens and hit[1] == cu_seqlens._version:
        return hit[2]
    full = torch.cat([cu_seqlens.new_zeros(1), cu_seqlens])
    ref = weakref.ref(cu_seqlens, lambda _r, key=key: _WITH_ZERO.pop(key, None))
    _WITH_ZERO[key] = (ref, cu_seqlens._version, full)
    return full


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens, inv_temp=None, zero_start=True,
                   attend_current=False):
    """cu_seqlens with its leading 0 when zero_start (the default), document ends only
    otherwise, as in the reference (sb_varlen/__init__.py:71-78).  The kernels always work from
    the form with the leading 0, and the schedule is cached per cu_seqlens tensor (for the form
    without the 0 too: its zero-prefixed copy is made once per tensor): pass the same tensor to every layer."""
    if not zero_start:
        cu_seqlens = _with_leading_zero(cu_seqlens)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return _apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)


def _apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
    if q.numel() == 0:
        # no tokens (or no heads): nothing to launch; empty results that stay in the graph
        return q * 0, q.sum(-1) * 0
    if not torch.is_grad_enabled():
        # no backward can follow: detached inputs tell the forward to keep no carry table
        q, k, v = q.detach(), k.detach(), v.detach()
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    """The reference's inner entry point (sb_varlen/__init__.py:81-82): cu_seqlens arrives with
    the leading 0 already stripped (document ends only)."""
    return _apply(q, k, v, _with_leading_zero(cu_seqlens), max_seqlens, inv_temp, attend_current)
