"""``CUDAAttention``: dense-phase softmax attention that also returns the full probability map.

Drop-in for the reference module of the same name (models/attention_cuda.py): constructor
``(config, attn_cpp=None, attn_handle=None)``, ``forward(query, key, value, mask)`` returning
``(out [B,H,L,d], P [B,H,L,L])``, both as transposed views of the feature-major / key-major buffers the
library fills (models/attention_cuda.py:32-36).  ``mask`` is ignored by this variant.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import _lib


class _DenseAttnFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key, value, mask, module):
        m = module
        _lib.use_current_stream(m, query.device)
        B, H, L, d = m.batch_size, m.num_heads, m.seq_len, m.emb_dim
        if tuple(query.shape) != (B, H, L, d):
            raise ValueError(f"query shape {tuple(query.shape)} does not match the handle ({B}, {H}, {L}, {d})")
        dev = query.device
        qt = _lib.transpose_last2(query)  # [B,H,d,L]
        k = key.contiguous()
        vt = _lib.transpose_last2(value)
        attn = torch.empty((B, H, L, L), dtype=torch.float32, device=dev)  # memory [key][query]
        out_t = torch.empty((B, H, d, L), dtype=torch.float32, device=dev)
        if m.with_mask:
            pen = (1e6 * (1.0 - mask.repeat(1, H))).to(torch.float32).contiguous()
            m.attn_cpp.attn_forward(m.attn_handle, qt.data_ptr(), k.data_ptr(), vt.data_ptr(), pen.data_ptr(),
                                    attn.data_ptr(), out_t.data_ptr())
        else:
            m.attn_cpp.attn_forward(m.attn_handle, qt.data_ptr(), k.data_ptr(), vt.data_ptr(), attn.data_ptr(),
                                    out_t.data_ptr())
        _lib.check_error("attn_forward")
        ctx.save_for_backward(qt, key, value, attn)
        ctx.set_materialize_grads(False)  # the gradient of the returned map is ignored (as in the reference)
        ctx.module = m
        return out_t.permute(0, 1, 3, 2), attn.permute(0, 1, 3, 2)

    @staticmethod
    def backward(ctx, grad_output, grad_weights):
        m = ctx.module
        _lib.use_current_stream(m, ctx.saved_tensors[0].device)
        qt, key, value, attn = ctx.saved_tensors
        B, H, L, d = m.batch_size, m.num_heads, m.seq_len, m.emb_dim
        dev = qt.device
        kt = _lib.transpose_last2(key)
        v = value.contiguous()
        if grad_output is None:  # only the returned map was used downstream: its gradient is ignored
            grad_output = torch.zeros(B, H, L, d, dtype=torch.float32, device=dev)
        got = _lib.transpose_last2(grad_output)
        dq_t = torch.empty((B, H, d, L), dtype=torch.float32, device=dev)
        dk_t = torch.empty((B, H, d, L), dtype=torch.float32, device=dev)
        dv_t = torch.empty((B, H, d, L), dtype=torch.float32, device=dev)
        # The ABI has three [NB, L, L] scratch arguments (models/attn.cu:273); this library needs none
        # of them, so nothing that size is allocated.
        none = None
        m.attn_cpp.attn_backward(m.attn_handle, qt.data_ptr(), kt.data_ptr(), v.data_ptr(), attn.data_ptr(),
                                 got.data_ptr(), none, none, none, dq_t.data_ptr(), dk_t.data_ptr(),
                                 dv_t.data_ptr())
        _lib.check_error("attn_backward")
        return dq_t.permute(0, 1, 3, 2), dk_t.permute(0, 1, 3, 2), dv_t.permute(0, 1, 3, 2), None, None


class _DenseAttentionBase(nn.Module):
    with_mask = False

    def __init__(self, config, attn_cpp=None, attn_handle=None):
        super().__init__()
        if attn_cpp is None or not attn_handle:
            raise _lib.SpionLibraryError(
                f"{type(self).__name__} needs the loaded HIP library and a handle from its init(); "
                "there is no fallback implementation"
            )
        self.emb_dim = config["head_dim"]
        self.num_heads = config["num_head"]
        self.seq_len = config["max_seq_len"]
        self.batch_size = config["batch_size"]
        self.num_batches = self.batch_size * self.num_heads
        self.attn_cpp = attn_cpp
        self.attn_handle = attn_handle
        self.attn_func = _DenseAttnFunction

    def forward(self, query, key, value, mask):
        return self.attn_func.apply(query, key, value, mask, self)


class CUDAAttention(_DenseAttentionBase):
    with_mask = False
