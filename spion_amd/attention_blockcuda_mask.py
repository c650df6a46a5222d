"""``CUDABlockMaskAttention``: sparse attention on a block mask with a key-padding mask.

Drop-in for the reference module of the same name (models/attention_blockcuda_mask.py): constructor
``(config, attn_cpp=None, attn_handle=None)``, ``forward(query, key, value, mask, mat)`` returning
``(out [B,H,L,d], 0)`` -- the probabilities are not handed back (models/attention_blockcuda_mask.py:62).
``mask`` is the [B, L] 0/1 key mask; it reaches the kernels as the additive penalty
``1e6 * (1 - mask)`` replicated per head (models/attention_blockcuda_mask.py:42-43).
"""
from __future__ import annotations

from .attention_blockcuda import _BlockAttentionBase


class CUDABlockMaskAttention(_BlockAttentionBase):
    with_mask = True

    def __init__(self, config, attn_cpp=None, attn_handle=None):
        super().__init__(config, attn_cpp, attn_handle)

    def forward(self, query, key, value, mask, mat):
        out, _ = self.run(query, key, value, mask, mat)
        return out, 0
