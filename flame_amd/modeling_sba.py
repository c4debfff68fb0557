"""SBA language model for the single-GPU training step (benchmark configuration 5).

Plain-PyTorch counterpart of custom_models/sba/modeling_sba.py:34-407 and config_sba.py:
pre-norm blocks [RMSNorm -> SBA -> +res -> RMSNorm -> SwiGLU MLP -> +res]
(modeling_sba.py:73-90, the non-fused branch :85-88), final norm, untied lm_head, labels
shifted left by one with the last position ignored (modeling_sba.py:391), mean
cross-entropy.  The reference builds its norm, MLP and loss from the `fla` package, which
is not part of the reference tree; the non-fused PyTorch equivalents are used
(nn.RMSNorm, explicit SwiGLU, F.cross_entropy).  MLP width follows fla's GatedMLP rule
for hidden_ratio=4: 2/3 * 4 * hidden rounded up to a multiple of 256 (2816 for 1024).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .sba_layer import SBA, fused_weight


@dataclass
class SBAConfig:
    # defaults = configs/sba_340m.json of the reference
    hidden_size: int = 1024
    num_hidden_layers: int = 24
    num_heads: int = 16
    hidden_ratio: int = 4
    intermediate_size: Optional[int] = None
    initializer_range: float = 0.006
    norm_eps: float = 1e-6
    vocab_size: int = 32000
    qkv_bias: bool = False
    num_kv_heads: Optional[int] = None
    window_size: Optional[int] = None
    tie_word_embeddings: bool = False

    def mlp_width(self) -> int:
        if self.intermediate_size is not None:
            return self.intermediate_size
        w = int(self.hidden_size * self.hidden_ratio * 2 / 3)
        return 256 * ((w + 255) // 256)


def _autocast_once(t: torch.Tensor) -> torch.Tensor:
    """Under autocast every nn.Linear casts its fp32 input by itself: the norm output that feeds
    q/k/v (or gate/up) would be cast three (two) times forward and its gradient as often backward.
    Casting it once here gives the linears the same bits."""
    if t.is_cuda and torch.is_autocast_enabled("cuda"):
        return t.to(torch.get_autocast_dtype("cuda"))
    return t


class _SwiGLU(torch.autograd.Function):
    """silu(g) * u on y = [g | u] (the output of the stacked gate/up product).  What autograd would do, except
    that the two halves of the gradient are written straight into one [.., 2*width] tensor - the shape the
    stacked product's backward wants - instead of being concatenated afterwards."""

    @staticmethod
    def forward(ctx, y):
        g, u = y.chunk(2, dim=-1)
        s = F.silu(g)
        ctx.save_for_backward(y, s)
        return s * u

    @staticmethod
    def backward(ctx, do):
        y, s = ctx.saved_tensors
        g, u = y.chunk(2, dim=-1)
        dy = torch.empty_like(y)
        dg, du = dy.chunk(2, dim=-1)
        torch.mul(do, s, out=du)
        torch.ops.aten.silu_backward.grad_input(do * u, g, grad_input=dg)
        return dy


def swiglu(y: torch.Tensor) -> torch.Tensor:
    if torch.compiler.is_compiling():       # the compiler fuses the plain form by itself
        g, u = y.chunk(2, dim=-1)
        return F.silu(g) * u
    return _SwiGLU.apply(y)


class SBAMLP(nn.Module):
    def __init__(self, cfg: SBAConfig):
        super().__init__()
        w = cfg.mlp_width()
        self.gate_proj = nn.Linear(cfg.hidden_size, w, bias=False)
        self.up_proj = nn.Linear(cfg.hidden_size, w, bias=False)
        self.down_proj = nn.Linear(w, cfg.hidden_size, bias=False)

    def forward(self, x):
        # gate and up in one [hidden, 2*width] product (see SBA.forward); the parameters stay gate_proj / up_proj
        return self.down_proj(swiglu(F.linear(x, fused_weight(x, self.gate_proj.weight, self.up_proj.weight))))


class SBABlock(nn.Module):
    def __init__(self, cfg: SBAConfig, layer_idx: int):
        super().__init__()
        self.attn_norm = nn.RMSNorm(cfg.hidden_size, eps=cfg.norm_eps)
        # every attention field the reference block forwards (modeling_sba.py:44-53): a num_kv_heads the layer
        # cannot do raises there instead of silently building full multi-head attention
        self.attn = SBA(hidden_size=cfg.hidden_size, num_heads=cfg.num_heads,
                        num_kv_heads=getattr(cfg, "num_kv_heads", None), qkv_bias=cfg.qkv_bias,
                        window_size=getattr(cfg, "window_size", None),
                        rope_theta=getattr(cfg, "rope_theta", None),
                        max_position_embeddings=getattr(cfg, "max_position_embeddings", None),
                        layer_idx=layer_idx)
        self.mlp_norm = nn.RMSNorm(cfg.hidden_size, eps=cfg.norm_eps)
        self.mlp = SBAMLP(cfg)

    def forward(self, x, **kwargs):
        h, _, _ = self.attn(_autocast_once(self.attn_norm(x)), **kwargs)
        x = x + h
        return x + self.mlp(_autocast_once(self.mlp_norm(x)))


class SBAModel(nn.Module):
    def __init__(self, cfg: SBAConfig):
        super().__init__()
        self.embeddings = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList([SBABlock(cfg, i) for i in range(cfg.num_hidden_layers)])
        self.norm = nn.RMSNorm(cfg.hidden_size, eps=cfg.norm_eps)

    def forward(self, input_ids, **kwargs):
        x = self.embeddings(input_ids)
        for layer in self.layers:
            x = layer(x, **kwargs)
        return self.norm(x)


class SBAForCausalLM(nn.Module):
    def __init__(self, cfg: SBAConfig):
        super().__init__()
        self.config = cfg
        self.model = SBAModel(cfg)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        self.apply(self._init_weights)
        if cfg.tie_word_embeddings:
            self.lm_head.weight = self.model.embeddings.weight

    def _init_weights(self, m):
        # modeling_sba.py:120-127: N(0, initializer_range) for Linear and Embedding
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, mean=0.0, std=self.config.initializer_range)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.Embedding):
            nn.init.normal_(m.weight, mean=0.0, std=self.config.initializer_range)

    def forward(self, input_ids, labels=None, **kwargs):
        h = self.model(input_ids, **kwargs)
        logits = self.lm_head(h)
        loss = None
        if labels is not None:
            shifted = torch.cat((labels[..., 1:], torch.full_like(labels[:, :1], -100)), 1)
            loss = F.cross_entropy(logits.view(shifted.numel(), -1).float(), shifted.view(-1), ignore_index=-100)
        return loss, logits

    def num_parameters(self, exclude_embeddings=False):
        n = sum(p.numel() for p in self.parameters())
        if exclude_embeddings:
            n -= self.model.embeddings.weight.numel()
        return n
