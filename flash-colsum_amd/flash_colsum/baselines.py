"""Eager attention column means that materialise the full attention matrix.

User-facing counterpart of the reference's baseline (reference:
flash_colsum/baselines.py:13-78).  It runs on whatever device its inputs live on and is
exported for comparisons only: `flash_colsum` never calls it.
"""
from typing import Optional

import torch


def naive_colsum(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
) -> torch.Tensor:
    """softmax(Q K^T * scale) averaged over heads and query rows -> (B, S_k).

    Causal alignment: key j is visible to query i iff j <= max(0, S_k - S_q) + i, i.e. all
    queries see the key prefix and the last S_q keys are lower-triangular
    (reference: baselines.py:49-62).  With `cls_len` only the first min(cls_len, S_q)
    query rows are averaged (reference: baselines.py:68-73).
    """
    s_q, d = query.shape[-2], query.shape[-1]
    s_k = key.shape[-2]
    if scale is None:
        scale = d ** -0.5
    logits = (query @ key.transpose(-2, -1)) * scale
    if is_causal:
        rows = torch.arange(s_q, device=query.device)[:, None] + max(0, s_k - s_q)
        cols = torch.arange(s_k, device=query.device)[None, :]
        logits = logits.masked_fill(cols > rows, float("-inf"))
    attn = torch.softmax(logits, dim=-1, dtype=torch.float32).to(query.dtype)
    if cls_len is not None and not is_causal:
        if cls_len <= 0:
            raise ValueError(f"cls_len must be positive, got {cls_len}")
        attn = attn[:, :, : min(int(cls_len), s_q)]
    return attn.mean(dim=(1, 2))


__all__ = ["naive_colsum"]
