"""Eager-torch CPU restatement of the reference's `naive_colsum`.  Test infrastructure.

Follows reference flash_colsum/baselines.py:35-78 step by step:
  scores = Q @ K^T * scale                              (baselines.py:42)
  causal: key j is visible to query i  <=>  j <= max(0, S_k - S_q) + i
          (baselines.py:49-62 builds the same set as "prefix columns all visible +
          lower-triangular window pasted at column S_k - S_q", and plain k <= q when
          S_k < S_q; the Triton launcher states the predicate directly,
          kernel_causal.py:39,57,113)
  softmax over keys in float32                          (baselines.py:66)
  optional restriction to the first min(cls_len, S_q) query rows (baselines.py:68-73)
  mean over heads and query rows                        (baselines.py:73,76)
The default scale is 1/sqrt(D) (baselines.py:38-39, ops.py:74-75).
"""
from typing import Optional

import torch


def visible(s_q: int, s_k: int, device=None) -> torch.Tensor:
    """Boolean (s_q, s_k) matrix of the aligned causal mask (baselines.py:49-62)."""
    k_past = max(0, s_k - s_q)
    i = torch.arange(s_q, device=device).view(s_q, 1)
    j = torch.arange(s_k, device=device).view(1, s_k)
    return j <= (i + k_past)


def naive_colsum(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
) -> torch.Tensor:
    """Column means of softmax(Q K^T * scale): (B, S_k), materialising the full matrix.

    Same operation sequence (and therefore the same cost profile) as the reference
    oracle, so it doubles as the reported CPU baseline.
    """
    _, _, s_q, d = query.shape
    s_k = key.shape[2]
    if scale is None:
        scale = 1.0 / (d ** 0.5)
    scores = torch.matmul(query, key.transpose(-1, -2)) * scale
    if is_causal:
        hidden = ~visible(s_q, s_k, device=query.device)
        scores = scores.masked_fill(hidden[None, None], float("-inf"))
    probs = torch.softmax(scores, dim=-1, dtype=torch.float32).to(query.dtype)
    if not is_causal and cls_len is not None:
        if cls_len <= 0:
            raise ValueError(f"cls_len must be positive, got {cls_len}")
        probs = probs[:, :, : min(int(cls_len), s_q), :]
    return probs.mean(dim=(1, 2))


def colsum_exact(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
    acc_dtype: torch.dtype = torch.float64,
    row_block: int = 1024,
) -> torch.Tensor:
    """Same quantity, one (batch, head, row block) at a time, accumulated in `acc_dtype`.

    The score matrix of one row block is (row_block, S_k), so memory stays bounded at the
    largest benchmark shapes.  Scores are computed in the input dtype's float32 upcast
    (exact products of fp16 values, fp32 BLAS accumulation) and the softmax and the
    running column sums in `acc_dtype`.  The result lives on the inputs' device.
    """
    b_n, h_n, s_q, d = query.shape
    s_k = key.shape[2]
    if scale is None:
        scale = 1.0 / (d ** 0.5)
    rows = s_q
    if not is_causal and cls_len is not None:
        if cls_len <= 0:
            raise ValueError(f"cls_len must be positive, got {cls_len}")
        rows = min(int(cls_len), s_q)
    k_past = max(0, s_k - s_q)
    dev = query.device  # runs wherever its inputs live (the tests use a GPU for the longest shapes)
    out = torch.zeros(b_n, s_k, dtype=acc_dtype, device=dev)
    j = torch.arange(s_k, device=dev).view(1, s_k)
    for b in range(b_n):
        for h in range(h_n):
            kt = key[b, h].to(torch.float32).t().contiguous()
            for r0 in range(0, rows, row_block):
                r1 = min(rows, r0 + row_block)
                s = (query[b, h, r0:r1].to(torch.float32) @ kt).to(acc_dtype) * scale
                if is_causal:
                    i = torch.arange(r0, r1, device=dev).view(-1, 1)
                    s = s.masked_fill(j > (i + k_past), float("-inf"))
                out[b] += torch.softmax(s, dim=-1).sum(dim=0)
    return out / (h_n * rows)


def colsum_ext_exact(
    query: torch.Tensor,
    key: torch.Tensor,
    scale: Optional[float] = None,
    is_causal: bool = False,
    cls_len: Optional[int] = None,
    k_past: Optional[int] = None,
    acc_dtype: torch.dtype = torch.float64,
    row_block: int = 1024,
) -> torch.Tensor:
    """Column means for the shapes the reference operator rejects (ops.py:65-66,79-87,93-97).

    The reference defines nothing here; the definition extends baselines.py:35-78 the way
    grouped-query attention is defined everywhere else:
      * key head of query head h is h // (H_q // H_k)  (the `repeat_interleave` of key heads);
      * the causal predicate j <= k_past + i (kernel_causal.py:39,57) applies to every batch
        entry alike, k_past defaulting to max(0, S_k - S_q) (kernel_causal.py:113);
      * `cls_len` restricts the mean to the first min(cls_len, S_q) query rows, also when causal;
      * S_q and S_k may differ without a mask.
    With H_q == H_k (and B == 1, cls_len None when causal) it is `colsum_exact`.
    """
    b_n, h_q, s_q, d = query.shape
    h_k, s_k = key.shape[1], key.shape[2]
    if key.shape[0] != b_n or key.shape[3] != d or h_q % h_k != 0:
        raise ValueError("query (B,Hq,Sq,D) and key (B,Hk,Sk,D) need the same B and D and Hq a multiple of Hk")
    grp = h_q // h_k
    if scale is None:
        scale = 1.0 / (d ** 0.5)
    rows = s_q
    if cls_len is not None:
        if cls_len <= 0:
            raise ValueError(f"cls_len must be positive, got {cls_len}")
        rows = min(int(cls_len), s_q)
    if k_past is None:
        k_past = max(0, s_k - s_q)
    dev = query.device
    out = torch.zeros(b_n, s_k, dtype=acc_dtype, device=dev)
    j = torch.arange(s_k, device=dev).view(1, s_k)
    for b in range(b_n):
        for h in range(h_q):
            kt = key[b, h // grp].to(torch.float32).t().contiguous()
            for r0 in range(0, rows, row_block):
                r1 = min(rows, r0 + row_block)
                s = (query[b, h, r0:r1].to(torch.float32) @ kt).to(acc_dtype) * scale
                if is_causal:
                    i = torch.arange(r0, r1, device=dev).view(-1, 1)
                    s = s.masked_fill(j > (i + k_past), float("-inf"))
                out[b] += torch.softmax(s, dim=-1).sum(dim=0)
    return out / (h_q * rows)
