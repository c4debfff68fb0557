"""SBA attention layer: counterpart of custom_models/sba/sba_layer.py:35-101.

Same parameters and the same forward contract (q/k/v projections, stick-breaking
attention with the default temperature, output projection; `rem` is discarded; no RoPE;
returns ``(o, None, past_key_values)``).  Two differences, both on purpose:

* `cu_seqlens` is honoured: the reference asserts it is None (sba_layer.py:86-87) and never
  reaches its varlen operator; here a packed batch ``[1, T, hidden]`` with ``cu_seqlens``
  is routed to ``sb_attn_varlen`` as ``[H, T, D]`` views (no copies).
* the head split/merge are strided views instead of ``.contiguous()`` copies
  (sba_layer.py:89-91): the kernels take strides.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn

from .stickbreaking_attention import sb_attn, sb_attn_varlen


class SBA(nn.Module):

    def __init__(self, hidden_size: int = 2048, num_heads: int = 32, num_kv_heads: Optional[int] = None,
                 qkv_bias: bool = False, window_size: Optional[int] = None,
                 rope_theta: Optional[float] = 10000., max_position_embeddings: Optional[int] = None,
                 layer_idx: int = None):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        if self.num_kv_heads != self.num_heads:
            # the reference passes q/k/v straight through, so kv_heads != heads cannot work there
            # either (sba_layer.py:89-93); say so instead of failing inside the kernel
            raise ValueError("SBA supports num_kv_heads == num_heads only")
        self.num_kv_groups = 1
        self.head_dim = hidden_size // num_heads
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.qkv_bias = qkv_bias
        self.window_size = window_size
        self.rope_theta = rope_theta
        self.max_position_embeddings = max_position_embeddings
        self.layer_idx = layer_idx

        self.q_proj = nn.Linear(hidden_size, hidden_size, bias=qkv_bias)
        self.k_proj = nn.Linear(hidden_size, self.kv_dim, bias=qkv_bias)
        self.v_proj = nn.Linear(hidden_size, self.kv_dim, bias=qkv_bias)
        self.o_proj = nn.Linear(hidden_size, hidden_size, bias=False)
        # tests swap these for the CPU oracle to check the model wiring
        self.attn_fn: Callable = sb_attn
        self.attn_varlen_fn: Callable = sb_attn_varlen

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_values=None, output_attentions: bool = False, use_cache: bool = False, **kwargs):
        assert attention_mask is None, "SBA does not support attention_mask yet"
        cu_seqlens = kwargs.get('cu_seqlens', None)
        B, T, _ = hidden_states.shape
        H, D = self.num_heads, self.head_dim
        q = self.q_proj(hidden_states)
        k = self.k_proj(hidden_states)
        v = self.v_proj(hidden_states)
        if cu_seqlens is not None:
            if B != 1:
                raise ValueError("cu_seqlens needs a packed batch of size 1")
            max_len = kwargs.get('max_seqlen', None)
            if max_len is None:
                max_len = T            # an upper bound is enough (the carry tables are sized from the documents)
            q, k, v = (x.view(T, H, D).transpose(0, 1) for x in (q, k, v))     # [H, T, D] views
            o, _ = self.attn_varlen_fn(q, k, v, cu_seqlens, max_len)
            o = o.transpose(0, 1).reshape(1, T, H * D)
        else:
            q, k, v = (x.view(B, T, H, D).transpose(1, 2) for x in (q, k, v))  # [B, H, T, D] views
            o, _ = self.attn_fn(q, k, v, None)
            o = o.transpose(1, 2).reshape(B, T, H * D)
        o = self.o_proj(o)
        return o, None, past_key_values
