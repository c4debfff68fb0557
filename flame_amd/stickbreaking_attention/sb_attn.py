"""Dense stick-breaking attention, [B, H, T, D].

Host-side mirror of custom_models/sba/stickbreaking_attention/sb_attn/__init__.py:16-64
(same function names, argument order, defaults and autograd contract); the Triton
launchers it called (sb_fwd.py:139-253, sb_bwd.py:163-297) are replaced by the C ABI
entry points sba_fwd / sba_bwd of libsba_mi355x.so.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from .. import _lib
from . import profiling


def _launch_fwd(q, k, v, inv_temp, attend_current, need_grad):
    lib = _lib.load()
    B, H, T, D = q.shape
    o = torch.empty_like(q)          # same strides as q (sb_fwd.py:144 does the same)
    rem = torch.empty((B, H, T), dtype=q.dtype, device=q.device)
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
    p.attend_current = int(bool(attend_current))
    p.scale = float(inv_temp)
    p.save_for_backward = int(need_grad)
    p.q, p.k, p.v, p.o = _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v), _lib.tensor4(o)
    p.rem = _lib.SbaVector(rem.data_ptr(), rem.stride(0), rem.stride(1))
    ws = None
    if need_grad:
        nbytes = lib.sba_workspace_bytes(C.byref(p))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), nbytes
    p.stream = torch.cuda.current_stream(q.device).cuda_stream
    profiling.mark("start")
    _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
    profiling.mark("fwd")
    return o, rem, ws


def _launch_bwd(do, drem, q, k, v, ws, inv_temp, attend_current):
    lib = _lib.load()
    B, H, T, D = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
    p.attend_current = int(bool(attend_current))
    p.scale = float(inv_temp)
    p.q, p.k, p.v = _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v)
    p.d_o = _lib.tensor4(do)
    if drem is not None:
        p.d_rem = _lib.SbaVector(drem.data_ptr(), drem.stride(0), drem.stride(1))
    p.dq, p.dk, p.dv = _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv)
    p.workspace, p.workspace_bytes = ws.data_ptr(), lib.sba_workspace_bytes(C.byref(p))
    p.stream = torch.cuda.current_stream(q.device).cuda_stream
    profiling.launch_bwd(lib, p)
    return dq, dk, dv


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, inv_temp: float,
                attend_current: bool = False):
        if not q.is_cuda:
            raise RuntimeError("stick-breaking attention runs on the GPU only (HIP kernels); "
                               "there is no CPU path")
        if not (q.dtype == k.dtype == v.dtype):
            raise TypeError("q, k, v must share a dtype")
        if not (q.shape == k.shape == v.shape) or q.dim() != 4:
            raise ValueError("q, k, v must all be [B, H, T, D]")
        need_grad = any(ctx.needs_input_grad[:3])
        q, k, v = _lib.usable(q), _lib.usable(k), _lib.usable(v)
        o, rem, ws = _launch_fwd(q, k, v, inv_temp, attend_current, need_grad)
        if need_grad:
            ctx.save_for_backward(q, k, v, ws)
        ctx.logit_scale = inv_temp
        ctx.attend_current = attend_current
        ctx.set_materialize_grads(False)
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, ws = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(q)
        do = _lib.usable(do)
        if drem is not None:
            drem = drem.contiguous()
        dq, dk, dv = _launch_bwd(do, drem, q, k, v, ws, ctx.logit_scale, ctx.attend_current)
        return dq, dk, dv, None, None


def sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False):
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_(q, k, v, inv_temp, attend_current=attend_current)


def sb_attn_(q, k, v, inv_temp, attend_current):
    return StickBreakingAttention.apply(q, k, v, inv_temp, attend_current)
