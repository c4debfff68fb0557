"""One single-GPU training step of the SBA language model (benchmark configuration 5):
bf16 autocast, fp32 master weights, AdamW (betas 0.9/0.95, eps 1e-15 and gradient
clipping 1.0 as in the reference's flame/models/fla.toml), one packed varlen sequence."""
from __future__ import annotations

import torch

from .modeling_sba import SBAConfig, SBAForCausalLM


def make_optimizer(model, lr=3e-4):
    return torch.optim.AdamW(model.parameters(), lr=lr, betas=(0.9, 0.95), eps=1e-15, weight_decay=0.1,
                             fused=True)


def train_step(model: SBAForCausalLM, opt, input_ids, labels, cu_seqlens=None, max_seqlen=None,
               clip: float = 1.0):
    opt.zero_grad(set_to_none=True)
    kwargs = {}
    if cu_seqlens is not None:
        kwargs = {"cu_seqlens": cu_seqlens, "max_seqlen": max_seqlen}
    with torch.autocast("cuda", dtype=torch.bfloat16):
        loss, _ = model(input_ids, labels=labels, **kwargs)
    loss.backward()
    gn = torch.nn.utils.clip_grad_norm_(model.parameters(), clip)
    opt.step()
    return loss.detach(), gn
