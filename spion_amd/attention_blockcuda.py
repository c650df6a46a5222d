"""``CUDABlockAttention``: sparse attention on a block mask, no key mask.

Drop-in for the reference module of the same name (models/attention_blockcuda.py): same constructor
``(config, attn_cpp, attn_handle)``, same ``forward(query, key, value, mask, mat)`` returning
``(out [B,H,L,d], P_flat [B*H*nnz])`` and the same autograd contract (gradients for query, key and value
only; the gradient of the returned probabilities is ignored, models/attention_blockcuda.py:73-112).
``attn_cpp`` is the ctypes library exporting init / attn_forward / attn_backward
(models/block_attn.cu:547-568), ``attn_handle`` the pointer its ``init`` returned.
"""
from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from . import _lib
from .csr import CsrCache


class _BlockAttnFunction(torch.autograd.Function):
    """The reference's function (models/attention_blockcuda.py:20-112) makes a transposed copy of K for the forward
    and of V for the backward because its ABI takes them that way, and its backward is not handed the forward's
    output.  Here every tensor stays row-major and autograd's saved ``out`` goes to the backward: the library's
    row-major entry points (spion_attn_forward_rowmajor / spion_attn_backward_rowmajor) take them as they are.
    ``attn_cpp`` (the drop-in with the reference's four symbols) is still what created the handle.

    The reference also starts with ``.contiguous()`` copies of query, key and value (models/attention_blockcuda.py:
    36-48), which arrive as [B,H,L,d] views of [B,L,H*d] projections (models/attention.py:136-139).  The strided
    entry points read the views in place, write ``out`` in the same interleaved layout (so that combine_heads,
    models/attention.py:131-134, is a view as well) and the gradients likewise: no copy on either side of the
    kernels.  (Head dimension 64 on tile patterns is served the same way; its kernels read row-major K and V a cache
    line per lane, slower than the transposed form the contiguous entry points use, but still cheaper than the
    copies.)"""

    @staticmethod
    def forward(ctx, query, key, value, mask, mat, module):
        m = module
        _lib.use_current_stream(m, query.device)
        idx = m.csr_cache.get(mat, m.block_size)
        nb_ = m.num_batches
        shape = m.head_shape
        if query.shape != shape:
            raise ValueError(f"query shape {tuple(query.shape)} does not match the handle {shape}")
        dev = query.device
        p_flat = torch.empty(nb_ * idx.nnz, dtype=torch.float32, device=dev)
        pen_ptr = None
        if m.with_mask:
            pen = (1e6 * (1.0 - mask.repeat(1, m.num_heads))).to(torch.float32).contiguous()  # [B, H*L]
            pen_ptr = pen.data_ptr()
        lay = None
        if m.reads_views and not (query.is_contiguous() and key.is_contiguous() and value.is_contiguous()):
            lay = _lib.head_layout(query)
            if lay is None or key.stride() != query.stride() or value.stride() != query.stride() \
                    or _lib.head_layout(key) is None or _lib.head_layout(value) is None:
                lay = None
        if lay is not None:
            q, k, v = query, key, value
            out = _empty_heads(shape, interleaved=query.stride(1) < query.stride(2), device=dev)
            lout = _lib.head_layout(out)
            _lib.core().spion_attn_forward_strided(
                m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr, p_flat.data_ptr(), out.data_ptr(),
                *idx.tail, m.num_heads, ctypes.addressof(lay), ctypes.addressof(lout))
        else:
            q, k, v = query.contiguous(), key.contiguous(), value.contiguous()
            out = torch.empty(shape, dtype=torch.float32, device=dev)
            _lib.core().spion_attn_forward_rowmajor(m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                                    p_flat.data_ptr(), out.data_ptr(), *idx.tail)
        _lib.check_error("attn_forward")
        # which kernel family serves THIS pattern (the handle may run other patterns before the backward)
        ctx.tiled = _lib.core().spion_last_path(m.attn_handle) == 1
        ctx.save_for_backward(q, k, v, p_flat, idx.offsets, idx.columns, idx.sum_mat, out)
        ctx.set_materialize_grads(False)  # the gradient of the returned probabilities is ignored anyway
        ctx.module = m
        ctx.nnz = idx.nnz
        ctx.tail = idx.tail  # the index tensors themselves are among the saved tensors
        ctx.strided = lay is not None
        if m.with_mask:
            ctx.mark_non_differentiable(p_flat)
        return out, p_flat

    @staticmethod
    def backward(ctx, grad_output, grad_weight):
        m = ctx.module
        _lib.use_current_stream(m, ctx.saved_tensors[0].device)
        q, k, v, p_flat, offsets, columns, sum_mat, out = ctx.saved_tensors
        dev = q.device
        n_total = m.num_batches * ctx.nnz
        if grad_output is None:  # only the probabilities were used downstream: their gradient is ignored
            grad_output = torch.zeros(m.batch_size, m.num_heads, m.seq_len, m.emb_dim, dtype=torch.float32, device=dev)
        core = _lib.core()
        if ctx.strided:
            go = grad_output
            if go.stride() != out.stride() or _lib.head_layout(go) is None:
                go = torch.empty_like(out).copy_(grad_output)  # preserves out's strides
            interleaved = q.stride(1) < q.stride(2)
            shape = tuple(q.shape)
            if _lib.adjacent_head_views(q, k, v):  # slices of one fused projection: the gradients likewise
                dq, dk, dv = _lib.empty_adjacent_heads(*shape, dev)
            else:
                dq, dk, dv = (_empty_heads(shape, interleaved, dev) for _ in range(3))
            lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
            core.spion_attn_backward_strided(
                m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), p_flat.data_ptr(), out.data_ptr(),
                go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), *ctx.tail, m.num_heads,
                ctypes.addressof(lin), ctypes.addressof(lout), ctypes.addressof(lgrad))
            _lib.check_error("attn_backward")
            return dq, dk, dv, None, None, None
        go = grad_output.contiguous()
        # Of the ABI's two [NB*nnz] scratch arguments (models/attention_blockcuda.py:83-84) the tile kernels use
        # neither and the element kernels only dS: nothing that size is allocated unless it is needed.
        scratch_ds = None
        if not ctx.tiled:
            scratch_ds = torch.empty(max(n_total, 1), dtype=torch.float32, device=dev)
        shape = m.head_shape
        dq = torch.empty(shape, dtype=torch.float32, device=dev)
        dk = torch.empty(shape, dtype=torch.float32, device=dev)
        dv = torch.empty(shape, dtype=torch.float32, device=dev)
        core.spion_attn_backward_rowmajor(
            m.attn_handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), p_flat.data_ptr(), out.data_ptr(), go.data_ptr(),
            scratch_ds.data_ptr() if scratch_ds is not None else None, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            *ctx.tail)
        _lib.check_error("attn_backward")
        return dq, dk, dv, None, None, None


def _empty_heads(shape, interleaved, device):
    """Uninitialised [B,H,L,d] tensor; ``interleaved``: in memory [B,L,H,d], i.e. [B,L,H*d] once the heads are merged."""
    B, H, L, d = shape
    if interleaved:
        return torch.empty((B, L, H, d), dtype=torch.float32, device=device).transpose(1, 2)
    return torch.empty(shape, dtype=torch.float32, device=device)


class _BlockAttentionBase(nn.Module):
    with_mask = False

    def __init__(self, config, attn_cpp, attn_handle):
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
        self.block_size = config["block_size"]
        self.num_batches = self.batch_size * self.num_heads
        self.num_blocks = int(self.seq_len / self.block_size)
        self.attn_cpp = attn_cpp
        self.attn_handle = attn_handle
        self.csr_cache = CsrCache(handle=attn_handle)
        self.attn_func = _BlockAttnFunction
        self.head_shape = (self.batch_size, self.num_heads, self.seq_len, self.emb_dim)
        _lib.core().spion_use_output_cache(attn_handle, 0)  # the backward is handed the output instead
        # every kernel family (tile, hybrid, element) reads [B,H,L,d] views of projections in place
        self.reads_views = self.emb_dim in (16, 32, 64, 128)


    def run(self, query, key, value, mask, mat):
        """(out, p_flat) through the compiled autograd node (csrc/autograd_node.cpp) -- the same steps as
        ``_BlockAttnFunction`` with the node, the saved tensors and the allocations on the C++ side of PyTorch, which
        takes a forward + backward of the L = 1024 tasks from 0.10 to 0.05 ms of host time -- or through the Python
        function when SPION_PY_NODE=1."""
        node = _lib.autograd_node()
        if node is None:
            return self.attn_func.apply(query, key, value, mask, mat, self)
        if query.shape != self.head_shape:
            raise ValueError(f"query shape {tuple(query.shape)} does not match the handle {self.head_shape}")
        idx = self.csr_cache.get(mat, self.block_size)
        pen = None
        if self.with_mask:
            pen = (1e6 * (1.0 - mask.repeat(1, self.num_heads))).to(torch.float32).contiguous()  # [B, H*L]
        index = query.device.index
        try:
            out, p_flat = node.sparse_attention(query, key, value, pen, idx.offsets, idx.columns, idx.sum_mat,
                                                self.attn_handle, idx.nnz, self.num_heads, self.reads_views,
                                                _lib._raw_stream(torch.cuda.current_device() if index is None else index))
        except RuntimeError as e:
            if str(e).startswith(("attn_forward:", "attn_backward:")):
                raise _lib.SpionLibraryError(str(e)) from None
            raise
        return out, p_flat


class CUDABlockAttention(_BlockAttentionBase):
    with_mask = False

    def forward(self, query, key, value, mask, mat):
        return self.run(query, key, value, mask, mat)
