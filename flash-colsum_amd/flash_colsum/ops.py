"""Public operator: attention column means without the attention matrix.

Drop-in for the reference's `flash_colsum` (reference: flash_colsum/ops.py:13-105): same
signature, same validation order and `ValueError`s, same result shapes and fp16 result
dtype.  The three Triton launchers it dispatched to are replaced by the gfx950 HIP
library bound in `_hip.py`.
"""
from typing import Optional

import torch

from . import _hip


def _validated(query, key, scale, is_causal, cls_len):
    """Checks in the reference's order (ops.py:59-97); returns (scale, cls_n)."""
    if query.ndim != 4 or key.ndim != 4:
        raise ValueError(f"Expected 4D tensors, got query.ndim={query.ndim}, key.ndim={key.ndim}")
    if query.device.type != "cuda":
        raise ValueError(f"Flash attention only supports CUDA tensors, got {query.device}")
    if cls_len is not None:
        if is_causal:
            raise ValueError("cls_len is only supported for non-causal attention")
        if cls_len <= 0:
            raise ValueError(f"cls_len must be positive, got {cls_len}")
    bq, hq, sq, dq = query.shape
    bk, hk, sk, dk = key.shape
    if scale is None:
        scale = dq ** -0.5
    if is_causal:
        if bq != 1 or bk != 1:
            raise ValueError(f"Causal attention currently only supports batch size 1, got B_q={bq}, B_k={bk}")
        if hq != hk or dq != dk:
            raise ValueError(
                f"Query and key must have same heads and head_dim, got H_q={hq}, H_k={hk}, D_q={dq}, D_k={dk}")
    elif (bq, hq, sq, dq) != (bk, hk, sk, dk):
        raise ValueError(
            "For non-causal attention, query and key must have same shape, got "
            f"query: {tuple(query.shape)}, key: {tuple(key.shape)}")
    return float(scale), (-1 if cls_len is None else int(cls_len))


def flash_colsum_f32(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
) -> torch.Tensor:
    """Same as `flash_colsum` but returns the kernels' fp32 means (no fp16 rounding)."""
    scale, cls_n = _validated(query, key, scale, is_causal, cls_len)
    if is_causal:
        return _hip.colsum_causal_f32(query, key, scale)
    return _hip.colsum_noncausal_f32(query, key, scale, cls_n)


def flash_colsum(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
) -> torch.Tensor:
    """Mean over heads and query rows of softmax(Q K^T * scale), per key position.

    query: (B, H, S, D); for `is_causal` (1, H, Q_len, D).
    key:   same shape as query; for `is_causal` (1, H, K_len, D), queries aligned to the
           last Q_len key positions.
    scale: defaults to 1/sqrt(D).
    cls_len: non-causal only; average over the first min(cls_len, S) query rows.
    Returns fp16 (B, S), or (1, K_len) for causal.  Raises ValueError for invalid input.
    """
    scale, cls_n = _validated(query, key, scale, is_causal, cls_len)
    if is_causal:
        return _hip._flash_colsum_causal(query, key, scale)
    if query.shape[0] == 1:
        return _hip._flash_colsum_non_batched(query, key, scale, CLS_N=cls_n)
    return _hip._flash_colsum_batched(query, key, scale, CLS_N=cls_n)


def flash_colsum_ext(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
    k_past: Optional[int] = None,
    out_dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """`flash_colsum` for the shapes the reference operator rejects (explicit opt-in: `flash_colsum`
    itself keeps raising for them, reference: flash_colsum/ops.py:65-66,79-87,93-97).

    * grouped-query / multi-query attention: key has H_k heads, H_q a multiple of H_k, query head h
      attends to key head h // (H_q // H_k); the mean runs over all H_q query heads;
    * causal with any batch size (query (B,H_q,Q_len,D), key (B,H_k,K_len,D), every batch entry aligned
      alike), and an explicit `k_past` (key j visible to query i  <=>  j <= k_past + i; default
      max(0, K_len - Q_len));
    * `cls_len` together with `is_causal`: the mean runs over the first min(cls_len, Q_len) query rows;
    * non-causal with S_q != S_k (cross-attention shape).
    Returns (B, S_k) in `out_dtype` (torch.float16 like the reference, or torch.float32).
    """
    if query.ndim != 4 or key.ndim != 4:
        raise ValueError(f"Expected 4D tensors, got query.ndim={query.ndim}, key.ndim={key.ndim}")
    if query.device.type != "cuda":
        raise ValueError(f"Flash attention only supports CUDA tensors, got {query.device}")
    if cls_len is not None and cls_len <= 0:
        raise ValueError(f"cls_len must be positive, got {cls_len}")
    bq, hq, sq, dq = query.shape
    bk, hk, sk, dk = key.shape
    if bq != bk or dq != dk:
        raise ValueError(f"Query and key must have same batch size and head_dim, got B_q={bq}, B_k={bk}, D_q={dq}, D_k={dk}")
    if hk < 1 or hq % hk != 0:
        raise ValueError(f"Query heads must be a multiple of key heads, got H_q={hq}, H_k={hk}")
    if k_past is not None and (not is_causal or k_past < 0):
        raise ValueError("k_past needs is_causal=True and a non-negative value")
    if out_dtype not in (torch.float16, torch.float32):
        raise ValueError(f"out_dtype must be torch.float16 or torch.float32, got {out_dtype}")
    if scale is None:
        scale = dq ** -0.5
    cls_n = -1 if cls_len is None else int(cls_len)
    if out_dtype == torch.float32:
        return _hip.colsum_general(query, key, float(scale), is_causal, cls_n, k_past)
    return _hip.colsum_general(query, key, float(scale), is_causal, cls_n, k_past, want_f16=True)[1]


def flash_colsum_topk(
    query: torch.Tensor,
    key: torch.Tensor,
    k: int,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
    sorted: bool = True,
    extended: bool = False,
):
    """The k most-attended key positions of every batch entry: `torch.topk` of the fp32 column means,
    computed on the GPU right behind them (no fp16 rounding in between, which at long contexts would
    flush most means to zero; no host synchronisation).

    Returns (values fp32 (B,k), indices int64 (B,k)); `sorted=True` orders them by descending value,
    `sorted=False` by ascending position.  Ties at the k-th value go to the lower position.
    `extended=True` accepts the shapes of `flash_colsum_ext`.
    """
    if extended:
        means = flash_colsum_ext(query, key, scale, is_causal, cls_len, out_dtype=torch.float32)
    else:
        means = flash_colsum_f32(query, key, scale, is_causal, cls_len)
    if not 1 <= int(k) <= means.shape[1]:
        raise ValueError(f"k must be in [1, {means.shape[1]}], got {k}")
    return _hip.topk_f32(means, int(k), sorted)


def flash_colsum_threshold(
    query: torch.Tensor,
    key: torch.Tensor,
    tau: float,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
):
    """Key positions whose fp32 column mean is >= tau: (indices int64 (B,S), counts int32 (B)); row b
    lists its positions, ascending, in its first counts[b] entries."""
    return _hip.threshold_f32(flash_colsum_f32(query, key, scale, is_causal, cls_len), float(tau))


__all__ = ["flash_colsum", "flash_colsum_f32", "flash_colsum_ext", "flash_colsum_topk", "flash_colsum_threshold"]
