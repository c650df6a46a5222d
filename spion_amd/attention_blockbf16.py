"""``BlockAttentionBF16``: sparse attention on a block mask for bf16 tensors (scale-up shapes).

The reference has no bf16 path; this module keeps the calling convention of its block modules
(models/attention_blockcuda_mask.py:21-103): ``forward(query, key, value, mask, mat)`` with
``query/key/value [B,H,L,d]`` and returns ``(out [B,H,L,d] bf16, 0)`` -- like the reference's key-mask
module it does not hand back the probabilities, which the kernels never write to memory.  The arithmetic
is the reference's sparse softmax (off-pattern keys count with logit 0 in the denominator) on bf16 inputs
with fp32 accumulation.  ``mask`` ([B, L] 0/1) is used only when the module was built with
``key_mask=True``; it reaches the kernels as ``1e6 * (1 - mask)`` per head.
"""
from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from . import _lib
from .csr import CsrCache


class _BlockBF16Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key, value, mask, mat, module):
        m = module
        _lib.use_current_stream(m, query.device)
        idx = m.csr_cache.get(mat, m.block_size)
        shape = (m.batch_size, m.num_heads, m.seq_len, m.emb_dim)
        if tuple(query.shape) != shape or tuple(key.shape) != shape or tuple(value.shape) != shape:
            raise ValueError(f"query/key/value shapes {tuple(query.shape)} do not match the handle {shape}")
        dev = query.device
        pen = None
        if m.key_mask:
            pen = (1e6 * (1.0 - mask.to(torch.float32))).repeat_interleave(m.num_heads, 0).contiguous()  # [B*H, L]
        pen_ptr = pen.data_ptr() if pen is not None else None
        lse = torch.empty((m.num_batches, m.seq_len), dtype=torch.float32, device=dev)
        # bf16 heads that are views of [B, L, H*d] projections (models/attention.py:136-139) are read in place and
        # the output is written interleaved the same way; anything else is converted and made contiguous first
        lay = None
        if all(t.dtype == torch.bfloat16 for t in (query, key, value)) and not (
                query.is_contiguous() and key.is_contiguous() and value.is_contiguous()):
            lay = _lib.head_layout(query)
            if lay is None or key.stride() != query.stride() or value.stride() != query.stride() \
                    or _lib.head_layout(key) is None or _lib.head_layout(value) is None:
                lay = None
        if lay is not None:
            q, k, v = query, key, value
            B, H, L, d = shape
            if query.stride(1) < query.stride(2):
                out = torch.empty((B, L, H, d), dtype=torch.bfloat16, device=dev).transpose(1, 2)
            else:
                out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
            lout = _lib.head_layout(out)
            m.lib.spion_block_bf16_attn_forward_strided(
                m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr, out.data_ptr(), lse.data_ptr(),
                *idx.tail, m.num_heads, ctypes.addressof(lay), ctypes.addressof(lout))
        else:
            q, k, v = (t.to(torch.bfloat16).contiguous() for t in (query, key, value))
            out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
            m.lib.spion_block_bf16_attn_forward(m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                                out.data_ptr(), lse.data_ptr(), *idx.tail)
        _lib.check_error("spion_block_bf16_attn_forward")
        ctx.save_for_backward(q, k, v, out, lse, idx.offsets, idx.columns, idx.sum_mat)
        ctx.pen = pen
        ctx.module = m
        ctx.tail = idx.tail
        ctx.strided = lay is not None
        return out

    @staticmethod
    def backward(ctx, grad_output):
        m = ctx.module
        _lib.use_current_stream(m, ctx.saved_tensors[0].device)
        q, k, v, out, lse, offsets, columns, sum_mat = ctx.saved_tensors
        pen = ctx.pen
        pen_ptr = pen.data_ptr() if pen is not None else None
        if ctx.strided:
            go = grad_output
            if go.dtype != torch.bfloat16 or go.stride() != out.stride() or _lib.head_layout(go) is None:
                go = torch.empty_like(out).copy_(grad_output)  # preserves out's strides
            B, H, L, d = q.shape
            if q.stride(1) < q.stride(2):
                dq, dk, dv = (torch.empty((B, L, H, d), dtype=torch.bfloat16, device=q.device).transpose(1, 2)
                              for _ in range(3))
            else:
                dq, dk, dv = (torch.empty((B, H, L, d), dtype=torch.bfloat16, device=q.device) for _ in range(3))
            lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
            m.lib.spion_block_bf16_attn_backward_strided(
                m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr, out.data_ptr(), lse.data_ptr(),
                go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), *ctx.tail, m.num_heads,
                ctypes.addressof(lin), ctypes.addressof(lout), ctypes.addressof(lgrad))
            _lib.check_error("spion_block_bf16_attn_backward_strided")
            return dq, dk, dv, None, None, None
        go = grad_output.to(torch.bfloat16).contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
        m.lib.spion_block_bf16_attn_backward(m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                             out.data_ptr(), lse.data_ptr(), go.data_ptr(), dq.data_ptr(),
                                             dk.data_ptr(), dv.data_ptr(), *ctx.tail)
        _lib.check_error("spion_block_bf16_attn_backward")
        return dq, dk, dv, None, None, None


class BlockAttentionBF16(nn.Module):
    def __init__(self, config, key_mask: bool = False, attn_handle=None):
        super().__init__()
        self.emb_dim = config["head_dim"]
        self.num_heads = config["num_head"]
        self.seq_len = config["max_seq_len"]
        self.batch_size = config["batch_size"]
        self.block_size = config["block_size"]
        self.num_batches = self.batch_size * self.num_heads
        self.key_mask = bool(key_mask)
        self.lib = _lib.core()  # raises when the HIP library has not been built: there is no fallback
        if not attn_handle:
            attn_handle = self.lib.spion_block_bf16_init(self.emb_dim, self.seq_len, self.num_batches, self.block_size)
            _lib.check_error("spion_block_bf16_init")
        self.attn_handle = attn_handle
        self.csr_cache = CsrCache(handle=attn_handle)
        self.reads_views = True  # bf16 heads that are views of projections are read in place

    def forward(self, query, key, value, mask, mat):
        return _BlockBF16Function.apply(query, key, value, mask, mat, self), 0
