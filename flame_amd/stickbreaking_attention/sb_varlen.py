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
from collections import OrderedDict

import torch

from .. import _lib
from . import profiling

_SCHEDULES: "OrderedDict[tuple, tuple]" = OrderedDict()
_MAX_CACHED = 16


def _schedule_for(cu_seqlens: torch.Tensor):
    """(cu int32 on device with leading 0, schedule on device, n_jobs, max_len, total)."""
    key = (cu_seqlens.data_ptr(), cu_seqlens.numel(), str(cu_seqlens.device), cu_seqlens._version,
           cu_seqlens.dtype)
    hit = _SCHEDULES.get(key)
    if hit is not None:
        _SCHEDULES.move_to_end(key)
        return hit
    cu_host = cu_seqlens.detach().to("cpu", torch.int32)   # one host sync per new packing
    if cu_host.numel() < 2 or int(cu_host[0]) != 0:
        raise ValueError("cu_seqlens must start with 0 and hold at least one document")
    lens = cu_host[1:] - cu_host[:-1]
    if bool((lens < 0).any()):
        raise ValueError("cu_seqlens must be non-decreasing")
    sched = _lib.build_schedule(cu_host)
    dev = cu_seqlens.device
    entry = (cu_host.to(dev), sched.to(dev), sched.shape[0], int(lens.max()), int(cu_host[-1]))
    _SCHEDULES[key] = entry
    while len(_SCHEDULES) > _MAX_CACHED:
        _SCHEDULES.popitem(last=False)
    return entry


def _params(q, k, v, sched_entry, inv_temp, attend_current):
    cu_dev, sched, n_jobs, max_len, total = sched_entry
    H, N, D = q.shape
    if total != N:
        raise ValueError(f"cu_seqlens ends at {total} but q has {N} tokens")
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = cu_dev.numel() - 1, H, max_len, N, D
    p.attend_current = int(bool(attend_current))
    p.scale = float(inv_temp)
    p.cu_seqlens, p.schedule, p.n_schedule = cu_dev.data_ptr(), sched.data_ptr(), n_jobs
    p.q, p.k, p.v = _lib.tensor3(q), _lib.tensor3(k), _lib.tensor3(v)
    p.stream = torch.cuda.current_stream(q.device).cuda_stream
    return p


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        if not q.is_cuda:
            raise RuntimeError("stick-breaking attention runs on the GPU only (HIP kernels); "
                               "there is no CPU path")
        if not (q.shape == k.shape == v.shape) or q.dim() != 3:
            raise ValueError("q, k, v must all be [H, total_tokens, D]")
        lib = _lib.load()
        need_grad = any(ctx.needs_input_grad[:3])
        q, k, v = _lib.usable(q), _lib.usable(k), _lib.usable(v)
        entry = _schedule_for(cu_seqlens)
        H, N, D = q.shape
        o = torch.empty_like(q)
        rem = torch.empty((H, N), dtype=q.dtype, device=q.device)
        ws = None
        if entry[2] > 0:
            p = _params(q, k, v, entry, inv_temp, attend_current)
            p.o = _lib.tensor3(o)
            p.rem = _lib.SbaVector(rem.data_ptr(), 0, rem.stride(0))
            p.save_for_backward = int(need_grad)
            if need_grad:
                nbytes = lib.sba_workspace_bytes(C.byref(p))
                ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
                p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
            profiling.mark("start")
            _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
            profiling.mark("fwd")
        if need_grad:
            ctx.save_for_backward(q, k, v, ws, cu_seqlens)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_seqlens
        ctx.attend_current = attend_current
        ctx.set_materialize_grads(False)
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        lib = _lib.load()
        q, k, v, ws, cu_seqlens = ctx.saved_tensors
        entry = _schedule_for(cu_seqlens)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        if entry[2] > 0:
            if do is None:
                do = torch.zeros_like(q)
            do = _lib.usable(do)
            p = _params(q, k, v, entry, ctx.logit_scale, ctx.attend_current)
            p.d_o = _lib.tensor3(do)
            if drem is not None:
                drem = drem.contiguous()
                p.d_rem = _lib.SbaVector(drem.data_ptr(), 0, drem.stride(0))
            p.dq, p.dk, p.dv = _lib.tensor3(dq), _lib.tensor3(dk), _lib.tensor3(dv)
            p.workspace, p.workspace_bytes = ws.data_ptr(), lib.sba_workspace_bytes(C.byref(p))
            profiling.launch_bwd(lib, p)
        return dq, dk, dv, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens, inv_temp=None, zero_start=True,
                   attend_current=False):
    if not zero_start:
        # the reference strips a leading 0 when zero_start; without one we prepend it, so
        # the kernels always see the same convention
        cu_seqlens = torch.cat([cu_seqlens.new_zeros(1), cu_seqlens])
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current)


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)
