"""cu_seqlens for a packed token row: the convention the reference's varlen collator
produces (flame/data.py:389-496), restated so that a packed batch can be fed to
``sb_attn_varlen`` / the SBA layer without flame's data pipeline.

Rules followed: int32; first entry 0; last entry = row length; document starts are the BOS
positions when the tokenizer has a BOS (a row not starting with BOS still starts a
document at 0), otherwise the positions after each EOS; an optional ``context_len``
re-chunks every document into pieces of at most that many tokens (data.py:475-492).
"""
from __future__ import annotations

from typing import Optional

import torch


def cu_seqlens_from_tokens(input_ids: torch.Tensor, bos_token_id: Optional[int] = None,
                           eos_token_id: Optional[int] = None,
                           context_len: Optional[int] = None) -> torch.Tensor:
    """input_ids: [1, T] or [T] packed row -> int32 cu_seqlens with a leading 0."""
    ids = input_ids.reshape(-1)
    T = ids.numel()
    if bos_token_id is not None:
        starts = torch.nonzero(ids == bos_token_id).flatten()
        if T > 0 and (starts.numel() == 0 or int(starts[0]) != 0):
            starts = torch.cat([starts.new_zeros(1), starts])
        cu = torch.cat([starts, starts.new_full((1,), T)])
    elif eos_token_id is not None:
        ends = torch.nonzero(ids == eos_token_id).flatten() + 1
        cu = torch.cat([ends.new_zeros(1), ends])
        if T == 0 or int(cu[-1]) != T:
            cu = torch.cat([cu, cu.new_full((1,), T)])
    else:
        raise ValueError("varlen packing without precomputed cu_seqlens needs a bos_token_id or an "
                         "eos_token_id to act as document separator")
    cu = cu.to(torch.int32)
    validate_cu_seqlens(cu, T)
    if context_len is not None:
        cu = split_by_context_len(cu, context_len)
    return cu


def validate_cu_seqlens(cu: torch.Tensor, total: int) -> None:
    """The checks of flame/data.py:459-473."""
    if cu.numel() < 2:
        raise ValueError(f"cu_seqlens must have at least start and end: {cu}")
    if not bool(torch.all(cu[1:] >= cu[:-1])):
        raise ValueError(f"cu_seqlens are not monotonically increasing: {cu}")
    if int(cu[0]) != 0:
        raise ValueError(f"cu_seqlens do not start at 0: {cu}")
    if int(cu[-1]) != total:
        raise ValueError(f"cu_seqlens do not end at total length {total}: {cu}")


def split_by_context_len(cu: torch.Tensor, context_len: int) -> torch.Tensor:
    """Re-chunk every document into pieces of at most context_len tokens."""
    total = int(cu[-1])
    pieces = [torch.arange(int(a), int(b), context_len, device=cu.device)
              for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()) if a < b]
    if not pieces:
        return torch.tensor([0, 0], dtype=torch.int32, device=cu.device)
    out = torch.cat(pieces + [torch.tensor([total], device=cu.device)]).to(torch.int32)
    return torch.unique(out)
