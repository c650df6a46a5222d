"""``CUDAAttention``: dense-phase softmax attention that also returns the full probability map.

Drop-in for the reference module of the same name (models/attention_cuda.py): constructor
``(config, attn_cpp=None, attn_handle=None)``, ``forward(query, key, value, mask)`` returning
``(out [B,H,L,d], P [B,H,L,L])``, both as transposed views of the feature-major / key-major buffers the
library fills (models/attention_cuda.py:32-36).  ``mask`` is ignored by this variant.
"""
from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from . import _lib


def _head_views(tensors):
    """The tensors as the strided entry points can take them (one common layout), or None."""
    lay = _lib.head_layout(tensors[0])
    if lay is None or any(t.stride() != tensors[0].stride() or _lib.head_layout(t) is None for t in tensors[1:]):
        return None
    return lay


def _empty_heads(shape, interleaved, device):
    B, H, L, d = shape
    if interleaved:  # memory [B, L, H, d]: merging the heads afterwards is a view
        return torch.empty((B, L, H, d), dtype=torch.float32, device=device).transpose(1, 2)
    return torch.empty(shape, dtype=torch.float32, device=device)


class _DenseAttnFunction(torch.autograd.Function):
    """The reference's function (models/attention_cuda.py:18-74) transposes Q and V for the forward and K and
    grad_output for the backward, because its ABI takes feature-major operands, and returns feature-major results
    as permuted views.  For head dimension 32 and sequences up to 16384, and head dimension 64 up to 2048, the
    library's strided entry points (spion_dense_forward_strided / spion_dense_backward_strided) take every tensor
    row-major -- also as views of [B, L, H*d] projections -- and nothing is transposed or copied; other shapes go
    through the reference's ABI."""

    @staticmethod
    def forward(ctx, query, key, value, mask, module):
        m = module
        _lib.use_current_stream(m, query.device)
        B, H, L, d = m.batch_size, m.num_heads, m.seq_len, m.emb_dim
        if tuple(query.shape) != (B, H, L, d):
            raise ValueError(f"query shape {tuple(query.shape)} does not match the handle ({B}, {H}, {L}, {d})")
        dev = query.device
        ctx.strided = False
        if m.reads_views:
            lay = _head_views((query, key, value))
            if lay is None:
                query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
                lay = _lib.head_layout(query)
            attn = torch.empty((B, H, L, L), dtype=torch.float32, device=dev)  # memory [key][query]
            out = _empty_heads((B, H, L, d), query.stride(1) < query.stride(2), dev)
            lout = _lib.head_layout(out)
            pen_ptr = None
            if m.with_mask:
                pen = (1e6 * (1.0 - mask.repeat(1, H))).to(torch.float32).contiguous()
                pen_ptr = pen.data_ptr()
            if m.emit_score_map and d == 32:
                # models/model_transformer.py:136-137 averages the returned maps over batch and heads; the kernel
                # does it while it writes them
                mean = torch.empty((L, L), dtype=torch.float32, device=dev)
                _lib.core().spion_dense_forward_strided_mean(
                    m.attn_handle, query.data_ptr(), key.data_ptr(), value.data_ptr(), pen_ptr, attn.data_ptr(),
                    out.data_ptr(), mean.data_ptr(), H, ctypes.addressof(lay), ctypes.addressof(lout))
                m.score_map = mean
            else:
                _lib.core().spion_dense_forward_strided(
                    m.attn_handle, query.data_ptr(), key.data_ptr(), value.data_ptr(), pen_ptr, attn.data_ptr(),
                    out.data_ptr(), H, ctypes.addressof(lay), ctypes.addressof(lout))
            _lib.check_error("attn_forward")
            if m.emit_score_map and d != 32:  # head dimension 64: one pass over the maps just written
                from .pattern import mean_score_map
                m.score_map = mean_score_map(attn.permute(0, 1, 3, 2))
            ctx.save_for_backward(query, key, value, attn, out)
            ctx.set_materialize_grads(False)
            ctx.module = m
            ctx.strided = True
            return out, attn.permute(0, 1, 3, 2)
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
        if m.emit_score_map:  # shapes the fused kernel does not serve: one pass over the maps just written
            from .pattern import mean_score_map
            m.score_map = mean_score_map(attn.permute(0, 1, 3, 2))
        ctx.save_for_backward(qt, key, value, attn)
        ctx.set_materialize_grads(False)  # the gradient of the returned map is ignored (as in the reference)
        ctx.module = m
        return out_t.permute(0, 1, 3, 2), attn.permute(0, 1, 3, 2)

    @staticmethod
    def backward(ctx, grad_output, grad_weights):
        m = ctx.module
        _lib.use_current_stream(m, ctx.saved_tensors[0].device)
        B, H, L, d = m.batch_size, m.num_heads, m.seq_len, m.emb_dim
        if ctx.strided:
            q, k, v, attn, out = ctx.saved_tensors
            dev = q.device
            if grad_output is None:  # only the returned map was used downstream: its gradient is ignored
                grad_output = torch.zeros(B, H, L, d, dtype=torch.float32, device=dev)
            go = grad_output
            if go.stride() != out.stride() or _lib.head_layout(go) is None:
                go = torch.empty_like(out).copy_(grad_output)  # keeps out's strides
            if _lib.adjacent_head_views(q, k, v):  # slices of one fused projection: the gradients likewise
                dq, dk, dv = _lib.empty_adjacent_heads(B, H, L, d, dev)
            else:
                dq, dk, dv = (_empty_heads((B, H, L, d), q.stride(1) < q.stride(2), dev) for _ in range(3))
            lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
            _lib.core().spion_dense_backward_strided(
                m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), attn.data_ptr(), out.data_ptr(),
                go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), H, ctypes.addressof(lin),
                ctypes.addressof(lout), ctypes.addressof(lgrad))
            _lib.check_error("attn_backward")
            return dq, dk, dv, None, None
        qt, key, value, attn = ctx.saved_tensors
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
        # shapes the strided entry points serve; everything else goes through the reference's ABI
        self.reads_views = (self.emb_dim == 32 and self.seq_len <= 16384) or (
            self.emb_dim == 64 and self.seq_len <= 2048)
        # When set, every forward also leaves ``self.score_map`` [L, L]: the mean of the returned maps over batch and
        # heads (what models/model_transformer.py:136-137 computes from them), taken while the maps are written.
        self.emit_score_map = False
        self.score_map = None

    def forward(self, query, key, value, mask):
        return self.attn_func.apply(query, key, value, mask, self)


class CUDAAttention(_DenseAttentionBase):
    with_mask = False
