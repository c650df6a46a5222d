"""``Attention``: multi-head attention layer that dispatches to the dense-phase or the sparse HIP path.

Mirrors the reference wrapper (models/attention.py:40-191): same constructor ``(config, inference=False)``,
``forward(X, mask, mat=None) -> (out, attn)``, ``reconstruct_for_blocksparse(config)`` and the four
static library loaders.  ``config`` keys read: transformer_dim, head_dim, num_head, max_seq_len,
block_size, batch_size, attention_dropout, task.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from . import _lib

# tasks whose inputs carry padding and therefore use the *_mask libraries (models/attention.py:11)
mask_task = ['lra-listops', 'lra-text', 'lra-news', 'lra-yelp', 'lra-text1', 'lra-news1', 'lra-yelp1',
             'lra-text2', 'lra-news2', 'lra-yelp2', 'lra-retrieval']


class SoftmaxAttention(nn.Module):
    """Plain PyTorch softmax attention with key mask and dropout (models/attention.py:13-38).

    Only used for the task the reference excludes from its native path; it is not a fallback for the
    HIP modules.
    """

    def __init__(self, config, inference=False):
        super().__init__()
        self.drop_attn = torch.nn.Dropout(p=config["attention_dropout"])
        self.head_dim = config["head_dim"]
        self.inference = inference

    def forward(self, Q, K, V, mask):
        dot = torch.matmul(Q, torch.transpose(K, -2, -1)) / math.sqrt(self.head_dim)
        dot = dot - 1e6 * (1 - mask[:, None, None, :])
        attn = self.drop_attn(nn.functional.softmax(dot, dim=-1))
        return torch.matmul(attn, V), attn


class _FusedQKV(torch.autograd.Function):
    """The three projections of models/attention.py:84-86 as one GEMM: X [B,L,dim] times the stacked weights gives one
    [B, L, 3, H, d] buffer whose slices are returned as the [B,H,L,d] heads (what split_heads, :136-139, makes of
    each projection).  The attention modules read such views in place and hand back gradients that are slices of one
    buffer again, so the backward is one GEMM for dX and one for the stacked weight gradient, without a copy."""

    @staticmethod
    def forward(ctx, X, wq, wk, wv, bq, bk, bv, H, d):
        B, L, dim = X.shape
        w = torch.cat((wq, wk, wv), 0)
        b = torch.cat((bq, bk, bv), 0)
        X2 = X.reshape(B * L, dim)
        qkv = torch.addmm(b, X2, w.t()).view(B, L, 3, H, d)
        ctx.save_for_backward(X2, w)
        ctx.dims = (B, H, L, d, dim)
        return tuple(qkv[:, :, i].transpose(1, 2) for i in range(3))

    @staticmethod
    def backward(ctx, dq, dk, dv):
        X2, w = ctx.saved_tensors
        B, H, L, d, dim = ctx.dims
        n = H * d
        if any(g is None for g in (dq, dk, dv)):
            z = next(g for g in (dq, dk, dv) if g is not None)
            dq, dk, dv = (torch.zeros_like(z) if g is None else g for g in (dq, dk, dv))
        if _lib.adjacent_head_views(dq, dk, dv):
            g2 = torch.as_strided(dq, (B * L, 3 * n), (3 * n, 1))
        else:
            g2 = torch.stack([g.transpose(1, 2) for g in (dq, dk, dv)], 2).reshape(B * L, 3 * n)
        dX = (g2 @ w).view(B, L, dim) if ctx.needs_input_grad[0] else None
        dW = g2.t() @ X2
        db = g2.sum(0)
        return (dX, dW[:n], dW[n:2 * n], dW[2 * n:], db[:n], db[n:2 * n], db[2 * n:], None, None)


class Attention(nn.Module):
    def __init__(self, config, inference=False):
        super().__init__()
        self.inference = inference
        self.dim = config["transformer_dim"]
        self.head_dim = config["head_dim"]
        self.num_head = config["num_head"]
        self.seq_len = config["max_seq_len"]
        self.block_size = config["block_size"]
        self.num_blocks = int(self.seq_len / self.block_size)

        # one GEMM for the three projections (same parameters, same state dict as the reference's three layers)
        self.fused_qkv = bool(config.get("fused_qkv", True))
        self.W_q = nn.Linear(self.dim, self.num_head * self.head_dim)
        self.W_k = nn.Linear(self.dim, self.num_head * self.head_dim)
        self.W_v = nn.Linear(self.dim, self.num_head * self.head_dim)

        if not inference:
            if config["task"] == "lra-pathfinder32-curv_contour_length_14":
                self.attn = SoftmaxAttention(config, inference)
            else:
                num_batches = config["num_head"] * config["batch_size"]
                if config["task"] in mask_task:
                    from .attention_cuda_mask import CUDAMaskAttention
                    attn_cpp = Attention._cuda_mask_compile_module()
                    handle = attn_cpp.init(config["head_dim"], config["max_seq_len"], num_batches)
                    _lib.check_error("attn_mask init")
                    self.attn = CUDAMaskAttention(config, attn_cpp, handle)
                else:
                    from .attention_cuda import CUDAAttention
                    attn_cpp = Attention._cuda_compile_module()
                    handle = attn_cpp.init(config["head_dim"], config["max_seq_len"], num_batches)
                    _lib.check_error("attn init")
                    self.attn = CUDAAttention(config, attn_cpp, handle)

        self.ff = nn.Linear(self.num_head * self.head_dim, self.dim)

    def forward(self, X, mask, mat=None):
        """Can be recorded into a HIP graph as a whole layer, forward and backward (tests/test_gpu_graph.py), under
        torch's usual rule for capturing a backward: warm up on a side stream and keep no autograd graph of a step
        that ran on the default stream alive (its AccumulateGrad nodes belong to the legacy stream, which a capture
        must not touch; breaking this rule ends in a crash inside capture_end on ROCm, not in an error message)."""
        if self.fused_qkv and X.dtype == torch.float32 and not torch.is_autocast_enabled():
            Q, K, V = _FusedQKV.apply(X, self.W_q.weight, self.W_k.weight, self.W_v.weight, self.W_q.bias,
                                      self.W_k.bias, self.W_v.bias, self.num_head, self.head_dim)
        else:
            Q = self.split_heads(self.W_q(X))
            K = self.split_heads(self.W_k(X))
            V = self.split_heads(self.W_v(X))
        # the kernels are fp32: leave autocast for the attention core (models/attention.py:88-92)
        with torch.autocast(device_type=X.device.type, enabled=False):
            if mat is None:
                attn_out, attn = self.attn(Q.float(), K.float(), V.float(), mask.float())
            else:
                attn_out, attn = self.block_attn(Q.float(), K.float(), V.float(), mask.float(), mat)
        attn_out = self.combine_heads(attn_out)
        return self.ff(attn_out), attn

    def reconstruct_for_blocksparse(self, config):
        """Switch the layer to the sparse path: load the block library, create its handle and the
        block module (models/attention.py:105-129)."""
        num_batches = int(config["num_head"] * config["batch_size"])
        if config["task"] in mask_task:
            from .attention_blockcuda_mask import CUDABlockMaskAttention
            cpp = Attention._blockcuda_mask_compile_module()
            handle = cpp.init(config["head_dim"], config["max_seq_len"], num_batches, config["block_size"])
            _lib.check_error("block_attn_mask init")
            self.block_attn = CUDABlockMaskAttention(config, cpp, handle)
        else:
            from .attention_blockcuda import CUDABlockAttention
            cpp = Attention._blockcuda_compile_module()
            handle = cpp.init(config["head_dim"], config["max_seq_len"], num_batches, config["block_size"])
            _lib.check_error("block_attn init")
            self.block_attn = CUDABlockAttention(config, cpp, handle)
        self.block_attn.to(next(self.parameters()).device)

    def combine_heads(self, X):
        X = X.transpose(1, 2)
        return X.reshape(X.size(0), X.size(1), self.num_head * self.head_dim)

    def split_heads(self, X):
        X = X.reshape(X.size(0), X.size(1), self.num_head, self.head_dim)
        return X.transpose(1, 2)

    # -- library loaders; argument counts as declared by the reference (models/attention.py:141-191)
    @staticmethod
    def _cuda_compile_module():
        return _lib.load_dropin("attn.so", n_init=3, n_fwd=6, n_bwd=12, trailing_int=False)

    @staticmethod
    def _blockcuda_compile_module():
        return _lib.load_dropin("block_attn.so", n_init=4, n_fwd=9, n_bwd=14, trailing_int=True)

    @staticmethod
    def _cuda_mask_compile_module():
        return _lib.load_dropin("attn_mask.so", n_init=3, n_fwd=7, n_bwd=12, trailing_int=False)

    @staticmethod
    def _blockcuda_mask_compile_module():
        return _lib.load_dropin("block_attn_mask.so", n_init=4, n_fwd=10, n_bwd=14, trailing_int=True)
