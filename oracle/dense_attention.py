"""CPU oracle: SPION dense-phase attention (the score-map producer).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

The reference computes it with cuBLAS 11 batched GEMMs (absent from the
reference tree; ``cublasGemmStridedBatchedEx``, restated from its published
column-major definition C = op(A).B) around two hand-written softmax kernels.
"""
from __future__ import annotations

import numpy as np


def dense_attention_forward(Q, K, V, key_penalty=None):
    """Q, K, V [NB, L, d] -> (O [NB, L, d], P [NB, L, L]) with P[h, i, j] over keys j.

    models/attn.cu:179-213: S = Q K^T; per query i (models/attn.cu:9-36):
    v = S*scale, m = max(-10, max_j v), P = exp(v-m)/sum_j exp(v-m); O = P V.
    Mask variant models/attn_mask.cu:44-73: v = S*scale - key_penalty[h, j].

    Pinned by: torch.softmax / scaled_dot_product_attention (tests); shift
    invariance makes the -10 initialiser immaterial unless every logit of a
    row is below -10 by more than the exponent range.
    """
    NB, L, d = Q.shape
    dt = Q.dtype
    scale = dt.type(np.float32(1.0) / np.sqrt(np.float32(d)))
    v = np.einsum("hid,hjd->hij", Q, K) * scale
    if key_penalty is not None:
        v = v - key_penalty[:, None, :].astype(dt)
    m = np.maximum(v.max(axis=-1, keepdims=True), dt.type(-10.0))
    e = np.exp(v - m)
    P = e / e.sum(axis=-1, keepdims=True)
    O = np.einsum("hij,hjd->hid", P, V)
    return O, P


def dense_attention_backward(Q, K, V, P, dO):
    """models/attn.cu:215-262: dP = dO V^T; t = dP*P; g = sum_j t;
    dS = (t - P g)*scale (models/attn.cu:67-87); dQ = dS K; dK = dS^T Q; dV = P^T dO.

    Pinned by: torch.autograd on ordinary softmax attention (tests).
    """
    dt = Q.dtype
    d = Q.shape[-1]
    scale = dt.type(np.float32(1.0) / np.sqrt(np.float32(d)))
    dP = np.einsum("hid,hjd->hij", dO, V)
    t = dP * P
    g = t.sum(axis=-1, keepdims=True)
    dS = (t - P * g) * scale
    dQ = np.einsum("hij,hjd->hid", dS, K)
    dK = np.einsum("hij,hid->hjd", dS, Q)
    dV = np.einsum("hij,hid->hjd", P, dO)
    return dQ, dK, dV
