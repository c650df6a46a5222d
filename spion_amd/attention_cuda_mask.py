"""``CUDAMaskAttention``: dense-phase attention with a key-padding mask.

Drop-in for the reference module of the same name (models/attention_cuda_mask.py); identical to
``CUDAAttention`` except that ``1e6 * (1 - mask)`` is subtracted from the logits of padded keys
(models/attention_cuda_mask.py:23-24, models/attn_mask.cu:44-73).
"""
from __future__ import annotations

from .attention_cuda import _DenseAttentionBase


class CUDAMaskAttention(_DenseAttentionBase):
    with_mask = True
