"""Dense stick-breaking attention, [B, H, T, D].

Host-side mirror of custom_models/sba/stickbreaking_attention/sb_attn/__init__.py:16-64
(same function names, argument order, defaults and autograd contract); the Triton
launchers it called (sb_fwd.py:139-253, sb_bwd.py:163-297) are replaced by the C ABI
entry points sba_fwd / sba_bwd of libsba_mi355x.so.
"""
from __future__ import annotations

import ctypes as C
import os
import math
from typing import Optional

import torch

from .. import _lib
from . import profiling
from .utils import custom_op


def _params(q, k, v, inv_temp, attend_current):
    B, H, T, D = q.shape
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.dtype_code(q.dtype)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
    p.attend_current = int(bool(attend_current))
    p.scale = float(inv_temp)
    p.q, p.k, p.v = _lib.tensor4(q), _lib.tensor4(k), _lib.tensor4(v)
    p.stream = _lib.current_stream_handle(q.device)
    return p


# The two sizes depend on dtype, shape and the two switches that route a problem to the generic kernels: asked of the
# library once per such key (a size query costs as much host time as a launch, and a training step asks twice per layer).
_SIZES = {}


def _size_key(q, what):
    return (what, q.dtype, tuple(q.shape), os.environ.get("SBA_FORCE_GENERIC"), os.environ.get("SBA_FORCE_GENERIC_BWD"))


def workspace_bytes(q, inv_temp=1.0) -> int:
    """What lives from the forward to the backward (the forward's carry table)."""
    if torch.compiler.is_compiling():
        B, H, T, D = q.shape
        return _lib.workspace_upper_bound(H, _lib.dense_columns(B, T))
    key = _size_key(q, 0)
    n = _SIZES.get(key)
    if n is None:
        n = _SIZES[key] = int(_lib.load().sba_workspace_bytes(C.byref(_params(q, q, q, inv_temp, False))))
    return n


def bwd_scratch_bytes(q, have_workspace=True) -> int:
    """What the backward needs for the duration of its call only (one table more when the forward
    kept none)."""
    if torch.compiler.is_compiling():
        B, H, T, D = q.shape
        return _lib.bwd_scratch_upper_bound(H, _lib.dense_columns(B, T), B * T, D)
    key = _size_key(q, 1 if have_workspace else 2)
    n = _SIZES.get(key)
    if n is None:
        p = _params(q, q, q, 1.0, False)
        p.workspace = 1 if have_workspace else None       # only NULL or not is looked at
        n = _SIZES[key] = int(_lib.load().sba_bwd_scratch_bytes(C.byref(p)))
    return n


# Same registered names as the reference (sb_fwd.py:177, sb_bwd.py:207); outputs are
# allocated by the caller and mutated, as there.
@custom_op("attn_fwd", mutates_args=("o", "rem", "ws"))
def _compileable_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, logit_scale: float,
                     attend_current: bool, save: bool, o: torch.Tensor, rem: torch.Tensor,
                     ws: torch.Tensor) -> None:
    lib = _lib.load()
    p = _params(q, k, v, logit_scale, attend_current)
    p.o = _lib.tensor4(o)
    p.rem = _lib.SbaVector(rem.data_ptr(), rem.stride(0), rem.stride(1))
    p.save_for_backward = int(save)
    if save:
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    profiling.mark("start")
    _lib.check(lib.sba_fwd(C.byref(p)), "sba_fwd")
    profiling.mark("fwd")


@custom_op("attn_bwd", mutates_args=("dq", "dk", "dv", "scratch"))
def _compileable_backward(do: torch.Tensor, dr: Optional[torch.Tensor], q: torch.Tensor, k: torch.Tensor,
                          v: torch.Tensor, ws: torch.Tensor, scratch: torch.Tensor, logit_scale: float,
                          attend_current: bool, dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor) -> None:
    lib = _lib.load()
    p = _params(q, k, v, logit_scale, attend_current)
    p.d_o = _lib.tensor4(do)
    if dr is not None:
        p.d_rem = _lib.SbaVector(dr.data_ptr(), dr.stride(0), dr.stride(1))
    p.dq, p.dk, p.dv = _lib.tensor4(dq), _lib.tensor4(dk), _lib.tensor4(dv)
    if ws.numel() > 16:                   # a 16-byte stand-in means: nothing was kept, recompute the carries
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    p.bwd_scratch, p.bwd_scratch_bytes = scratch.data_ptr(), scratch.numel()
    profiling.launch_bwd(lib, p)


def attention_weights(q, k, inv_temp=None, attend_current=False):
    """The attention weights A_ij as float32 [B, H, T, T] (zero where j may not be attended): what the reference's
    forward returns as `W` under `return_attention=True` (sb_fwd.py:141-172).  For inspection and tests: a
    vector-ALU kernel, T x T floats per head."""
    if not q.is_cuda:
        raise RuntimeError("stick-breaking attention runs on the GPU only (HIP kernels); there is no CPU path")
    if q.shape != k.shape or q.dim() != 4 or q.dtype != k.dtype:
        raise ValueError("q, k must both be [B, H, T, D] of one dtype")
    _lib.check_supported(q)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    B, H, T, _ = q.shape
    W = torch.zeros((B, H, T, T), dtype=torch.float32, device=q.device)
    if W.numel():
        q, k = _lib.usable(q.detach()), _lib.usable(k.detach())
        p = _params(q, k, k, inv_temp, attend_current)
        _lib.check(_lib.load().sba_attention_weights(C.byref(p), W.data_ptr()), "sba_attention_weights")
    return W


def _fwd(q, k, v, logit_scale, attend_current=False, no_grad=False, return_attention=False):
    if return_attention:                 # the reference's debug output rides along as a fourth result
        return (*_fwd(q, k, v, logit_scale, attend_current, no_grad), attention_weights(q, k, logit_scale, attend_current))
    o = torch.empty_like(q)              # same strides as q (sb_fwd.py:144 does the same)
    rem = torch.empty(q.shape[:-1], dtype=q.dtype, device=q.device)
    # above the workspace budget nothing is kept and the backward recomputes the carries (_lib.recompute_carries)
    nbytes = 16 if no_grad else max(workspace_bytes(q), 16)
    keep = not (no_grad or _lib.recompute_carries(nbytes))
    if not keep:
        nbytes = 16
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    _compileable_fwd(q, k, v, float(logit_scale), bool(attend_current), keep, o, rem, ws)
    return o, rem, ws


def _bwd(do, dr, q, k, v, ws, logit_scale, attend_current=False):
    dq, dk, dv = _lib.empty_grads_like(q, k, v)     # one allocation when q, k, v are slices of one tensor
    # freed when this call returns: only the forward's table is kept between the two directions
    scratch = torch.empty(max(bwd_scratch_bytes(q, ws.numel() > 16), 16), dtype=torch.uint8, device=q.device)
    _compileable_backward(do, dr, q, k, v, ws, scratch, float(logit_scale), bool(attend_current), dq, dk, dv)
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
        if not (q.device == k.device == v.device):
            raise ValueError("q, k, v must be on the same device")
        if not (q.shape == k.shape == v.shape) or q.dim() != 4:
            raise ValueError("q, k, v must all be [B, H, T, D]")
        _lib.check_supported(q)
        no_grad = not any(ctx.needs_input_grad[:3])
        ctx.head_dim = q.shape[-1]
        Dp = _lib.matrix_core_head_dim(q)
        q, k, v = (_lib.usable(_lib.pad_head_dim(x, Dp)) for x in (q, k, v))
        o, rem, ws = _fwd(q, k, v, inv_temp, attend_current, no_grad)
        ctx.save_for_backward(q, k, v, ws)
        ctx.logit_scale = inv_temp
        ctx.attend_current = attend_current
        ctx.set_materialize_grads(False)
        return _lib.cut_head_dim(o, ctx.head_dim), rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, ws = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(q)
        do = _lib.usable(_lib.pad_head_dim(do, q.shape[-1]))
        if drem is not None:
            drem = drem.contiguous()
        dq, dk, dv = _bwd(do, drem, q, k, v, ws, ctx.logit_scale, ctx.attend_current)
        return (*(_lib.cut_head_dim(g, ctx.head_dim) for g in (dq, dk, dv)), None, None)


def sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False):
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_(q, k, v, inv_temp, attend_current=attend_current)


def sb_attn_(q, k, v, inv_temp, attend_current):
    if q.numel() == 0:
        # nothing to launch (an empty batch or a zero-length sequence): empty results that stay in the graph
        return q * 0, q.sum(-1) * 0
    if not torch.is_grad_enabled():
        # no backward can follow: detached inputs tell the forward to keep no carry table
        q, k, v = q.detach(), k.detach(), v.detach()
    return StickBreakingAttention.apply(q, k, v, inv_temp, attend_current)
