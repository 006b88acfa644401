"""flash_colsum for AMD Instinct MI355X (gfx950).

Same public surface as the reference package (reference: flash_colsum/__init__.py:5-10):
`flash_colsum` is the fused operator, `naive_colsum` the eager baseline that materialises
the attention matrix.  `flash_colsum_f32` additionally exposes the kernels' fp32 means, `flash_colsum_ext` the shapes the
reference operator rejects (grouped key heads, batched causal calls, causal `cls_len`).
"""
from .ops import flash_colsum, flash_colsum_ext, flash_colsum_f32, flash_colsum_threshold, flash_colsum_topk
from .baselines import naive_colsum

__version__ = "1.0.0"
__all__ = ["flash_colsum", "flash_colsum_ext", "flash_colsum_f32", "flash_colsum_threshold", "flash_colsum_topk",
           "naive_colsum"]
