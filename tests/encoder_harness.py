"""Harness for benchmark configuration 3: a 2-layer pre-LN Transformer encoder for sequence classification
around the attention layer under test.

It restates the structure the reference trains (models/model_transformer.py:17-145 embeddings + layers + final
norm, models/model_LRA.py:8-71 mean pooling + MLP head + cross entropy; AdamW as in main_conv_ff.py:451-455) in
plain torch.nn; only the attention layer is the product (``spion_amd.Attention``) or, for the reference run, the
CPU oracle.  Test / benchmark infrastructure, not part of the package.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn


class OracleAttention(nn.Module):
    """Same parameters and interface as ``spion_amd.Attention`` (models/attention.py:40-103), attention core
    computed by the oracle's dense PyTorch statement on whatever device / dtype the module lives on."""

    def __init__(self, config):
        super().__init__()
        self.dim = config["transformer_dim"]
        self.head_dim = config["head_dim"]
        self.num_head = config["num_head"]
        self.block_size = config["block_size"]
        self.use_key_mask = config["use_key_mask"]
        self.W_q = nn.Linear(self.dim, self.num_head * self.head_dim)
        self.W_k = nn.Linear(self.dim, self.num_head * self.head_dim)
        self.W_v = nn.Linear(self.dim, self.num_head * self.head_dim)
        self.ff = nn.Linear(self.num_head * self.head_dim, self.dim)

    def _split(self, X):
        return X.reshape(X.size(0), X.size(1), self.num_head, self.head_dim).transpose(1, 2)

    def forward(self, X, mask, mat=None):
        from oracle import sparse_attention as osa

        Q, K, V = self._split(self.W_q(X)), self._split(self.W_k(X)), self._split(self.W_v(X))
        key_mask = mask.to(X.dtype) if self.use_key_mask else None
        L = X.size(1)
        if mat is None:
            pattern = torch.ones(L, L, dtype=X.dtype, device=X.device)
        else:
            bs = self.block_size
            pattern = mat.to(X.dtype).repeat_interleave(bs, 0).repeat_interleave(bs, 1)
        out, attn = osa.dense_masked_attention(Q, K, V, pattern, key_mask)
        out = out.transpose(1, 2).reshape(X.size(0), L, self.num_head * self.head_dim)
        return self.ff(out), attn


class EncoderLayer(nn.Module):
    def __init__(self, config, attention_cls):
        super().__init__()
        d, hid = config["transformer_dim"], config["transformer_hidden_dim"]
        self.norm1 = nn.LayerNorm(d)
        self.mha = attention_cls(config)
        self.norm2 = nn.LayerNorm(d)
        self.mlpblock = nn.Sequential(nn.Linear(d, hid), nn.GELU(), nn.Linear(hid, d))

    def forward(self, X, mask, mat=None):
        out, attn = self.mha(self.norm1(X), mask, mat)
        X = out + X
        return self.mlpblock(self.norm2(X)) + X, attn


class EncoderForSC(nn.Module):
    """Token + learned position embeddings, ``num_layers`` pre-LN layers, final LayerNorm * mask, mean pooling,
    Linear-ReLU-Linear head, per-sample cross entropy."""

    def __init__(self, config, attention_cls):
        super().__init__()
        d = config["transformer_dim"]
        self.num_layers = config["num_layers"]
        self.word_embeddings = nn.Embedding(config["vocab_size"], d)
        self.position_embeddings = nn.Embedding(config["max_seq_len"], d)
        nn.init.normal_(self.word_embeddings.weight, std=0.02)
        nn.init.normal_(self.position_embeddings.weight, std=0.02)
        self.layers = nn.ModuleList([EncoderLayer(config, attention_cls) for _ in range(self.num_layers)])
        self.norm = nn.LayerNorm(d)
        self.head = nn.Sequential(nn.Linear(d, config["transformer_hidden_dim"]), nn.ReLU(),
                                  nn.Linear(config["transformer_hidden_dim"], config["num_classes"]))

    def forward(self, input_ids, mask, label, mat_lst=None, is_attn=False):
        B, L = input_ids.shape
        pos = torch.arange(L, device=input_ids.device)[None, :].expand(B, L)
        X = self.word_embeddings(input_ids) + self.position_embeddings(pos)
        attn_lst = []
        for idx, layer in enumerate(self.layers):
            if mat_lst is None:
                core = getattr(layer.mha, "attn", None)
                fused = is_attn and hasattr(core, "emit_score_map")  # the HIP modules average while they write the maps
                if fused:
                    core.emit_score_map = True
                X, attn = layer(X, mask)
                if fused:
                    core.emit_score_map = False
                    attn_lst.append(core.score_map)
                elif is_attn:  # models/model_transformer.py:136-137: mean over batch, then over heads
                    attn_lst.append(torch.mean(torch.mean(attn, dim=0), dim=0))
            else:
                X, attn = layer(X, mask, mat_lst[0][idx])
        X = self.norm(X) * mask[:, :, None].to(X.dtype)
        pooled = X.mean(dim=1)
        scores = self.head(pooled)
        loss = nn.functional.cross_entropy(scores, label, reduction="none")
        self.last_accu = (scores.argmax(dim=-1) == label).to(torch.float32)  # models/model_LRA.py:62-63
        return loss, attn_lst

    def outputs(self, input_ids, mask, label, mat_lst=None):
        """The dict the reference's task model returns (models/model_LRA.py:52-71): per-sample loss and accuracy."""
        loss, _ = self.forward(input_ids, mask, label, mat_lst)
        return {"loss": loss, "accu": self.last_accu}


def model_config(L=1024, batch=256, block_size=32, key_mask=False, threshold=0.96):
    """Dimensions of the reference's image task (config.py:126-146)."""
    return {
        "embedding_dim": 64, "transformer_dim": 64, "transformer_hidden_dim": 128, "head_dim": 32, "num_head": 2,
        "num_layers": 2, "vocab_size": 256, "max_seq_len": L, "dropout_prob": 0.0, "attention_dropout": 0.0,
        "num_classes": 10, "block_size": block_size, "batch_size": batch, "density": 0.04, "threshold": threshold,
        "task": "lra-text" if key_mask else "lra-image", "use_key_mask": key_mask,
    }


def make_optimizer(model, lr=1e-4, weight_decay=0.0):
    return torch.optim.AdamW(model.parameters(), lr=lr, betas=(0.9, 0.999), eps=1e-6, weight_decay=weight_decay)


def synthetic_batch(config, seed=0, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    B, L = config["batch_size"], config["max_seq_len"]
    ids = torch.randint(0, config["vocab_size"], (B, L), generator=g)
    labels = torch.randint(0, config["num_classes"], (B,), generator=g)
    if config["use_key_mask"]:
        lens = torch.randint(L // 2, L + 1, (B,), generator=g)
        mask = (torch.arange(L)[None, :] < lens[:, None]).to(torch.float32)
    else:
        mask = torch.ones(B, L)
    return ids.to(device), mask.to(device), labels.to(device)
