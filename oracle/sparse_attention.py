"""CPU oracle: SPION sparse attention on an element-CSR pattern (forward + backward).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Two independent statements of the same mathematics live here:

* ``csr_*``: a literal, step-by-step restatement of the reference's native
  pipeline (SDDMM -> row softmax -> SpMM and its backward) on CSR arrays, in
  numpy, in the precision the caller picks (float64 is the ground truth the
  GPU results are compared to).
* ``dense_masked_attention``: the dense PyTorch formulation (off-pattern
  logits are 0, not -inf) whose autograd gives the backward.  It is also the
  CPU timing baseline.

Parity status of every function is recorded in its docstring ("pinned by").
The reference ships no tests or golden vectors for this path, and its
arithmetic lives in cuSPARSE 11 (CUDA 11.7.1: cusparseSDDMM / cusparseSpMM),
which is absent from the reference tree; those two routines are restated
from their published definitions (C = (A.B) o pattern; C = A_csr.B).
"""
from __future__ import annotations

import numpy as np


# --------------------------------------------------------------------------
# CSR construction
# --------------------------------------------------------------------------
def build_csr_from_block_mask(mat: np.ndarray, block_size: int):
    """Element-level CSR of a block mask upsampled by ``block_size``.

    Follows models/attention_blockcuda.py:26-43 (and the identical
    models/attention_blockcuda_mask.py:26-36):
      sum_mat[i]  = block_size * sum_j mat[i // bs, j]
      Offsets     = exclusive prefix sum of sum_mat, length L+1
      Columns     = column index of every non-zero of the nearest-neighbour
                    upsampled mask in row-major order (one head's worth; the
                    reference then repeats it NB times).
    Any non-zero entry of ``mat`` counts as set for Columns (``nonzero()``),
    while sum_mat sums the values; the two agree for 0/1 masks, which is all
    the reference produces.

    Pinned by: brute-force double loop in tests (tests/test_oracle_sparse.py).
    """
    mat = np.asarray(mat)
    nb = mat.shape[0]
    assert mat.shape == (nb, nb)
    bs = int(block_size)
    L = nb * bs
    row_counts = mat.astype(np.int64).sum(axis=1) * bs          # per block row
    sum_mat = np.repeat(row_counts, bs).astype(np.int32)         # [L]
    offsets = np.zeros(L + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(sum_mat)
    dense = np.repeat(np.repeat(mat != 0, bs, axis=0), bs, axis=1)
    columns = np.nonzero(dense)[1].astype(np.int32)
    return sum_mat, offsets, columns


def csr_from_dense_pattern(pattern: np.ndarray):
    """CSR arrays (sum_mat, offsets, columns) of an arbitrary [L, L] 0/1 pattern.

    This is what models/attention_blockcuda_mask.py:26-36 yields with
    ``block_size == 1`` (upsample factor 1), i.e. the element-sparse case.
    """
    pattern = np.asarray(pattern) != 0
    sum_mat = pattern.sum(axis=1).astype(np.int32)
    offsets = np.zeros(pattern.shape[0] + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(sum_mat)
    columns = np.nonzero(pattern)[1].astype(np.int32)
    return sum_mat, offsets, columns


def csr_row_index(offsets: np.ndarray) -> np.ndarray:
    """Row index of every CSR entry."""
    counts = np.diff(offsets.astype(np.int64))
    return np.repeat(np.arange(len(counts), dtype=np.int64), counts)


# --------------------------------------------------------------------------
# Literal CSR pipeline (numpy)
# --------------------------------------------------------------------------
def csr_sddmm(A: np.ndarray, B: np.ndarray, offsets, columns) -> np.ndarray:
    """values[h, k] = sum_t A[h, row(k), t] * B[h, col(k), t].

    The sampled dense-dense product the reference gets from cusparseSDDMM
    (models/block_attn.cu:145-224, called at :459 with A=Q, B=K^T and at :498
    with A=dO, B=V^T).  ``B`` is given here un-transposed, [NB, L, d].

    Pinned by: dense ``A @ B^T`` masked with the pattern (tests).
    """
    rows = csr_row_index(offsets)
    cols = np.asarray(columns, dtype=np.int64)
    return np.einsum("hkt,hkt->hk", A[:, rows, :], B[:, cols, :])


def csr_scale_softmax(values: np.ndarray, offsets, sum_mat, seq_len: int,
                      scale: float, key_penalty: np.ndarray | None = None,
                      columns=None) -> np.ndarray:
    """Row softmax of the reference, in which every off-pattern logit is 0.

    Without ``key_penalty`` follows models/block_attn.cu:33-88:
        v = S*scale; m = max(-100, max_k v); Z = sum_k exp(v-m) + (L-n_i)*exp(-m)
        r = 1/Z;  P = 0 if r == 0 else exp(v-m)*r
    With ``key_penalty`` [NB, L] (0 or 1e6) follows models/block_attn_mask.cu:88-140:
        v = S*scale - key_penalty[h, col_k];  m = max(0, max_k v);  rest the same.
    The ``r == 0`` guard fires when Z overflows to +inf in the working
    precision (fp32: row maximum below about -88.7 with L > n_i).

    Pinned by: (i) full pattern (n_i = L) equals an ordinary softmax;
    (ii) sum_k P_ik = 1 - (L - n_i) exp(-m)/Z; (iii) the dense formulation
    ``dense_masked_attention`` below, an independent statement; (iv) a
    scalar re-implementation of the serial kernel
    models/block_attn_mask.cu:28-66 on tiny inputs (tests).
    """
    values = np.asarray(values)
    dt = values.dtype
    NB, n = values.shape
    rows = csr_row_index(offsets)
    L = int(seq_len)
    v = values * dt.type(scale)
    if key_penalty is not None:
        cols = np.asarray(columns, dtype=np.int64)
        v = v - key_penalty[:, cols].astype(dt)
        m0 = dt.type(0.0)
    else:
        m0 = dt.type(-100.0)
    m = np.full((NB, L), m0, dtype=dt)
    if n:
        np.maximum.at(m, (slice(None), rows), v)
    e = np.exp(v - m[:, rows])
    Z = np.zeros((NB, L), dtype=dt)
    if n:
        np.add.at(Z, (slice(None), rows), e)
    with np.errstate(over="ignore", divide="ignore"):
        Z = Z + (L - np.asarray(sum_mat, dtype=dt))[None, :] * np.exp(-m)
        r = dt.type(1.0) / Z
    P = e * r[:, rows]
    P[(r == 0)[:, rows]] = 0
    return P.astype(dt)


def csr_spmm(values: np.ndarray, B: np.ndarray, offsets, columns) -> np.ndarray:
    """C[h, i, :] = sum_{k in row i} values[h, k] * B[h, col(k), :].

    cusparseSpMM, non-transposed (models/block_attn.cu:236-393; forward call
    :478 gives O = P.V, backward call :516 gives dQ = dS.K).
    Pinned by: dense matmul with the scattered matrix (tests).
    """
    rows = csr_row_index(offsets)
    cols = np.asarray(columns, dtype=np.int64)
    NB, L, d = B.shape
    C = np.zeros((NB, len(offsets) - 1, d), dtype=values.dtype)
    np.add.at(C, (slice(None), rows), values[:, :, None] * B[:, cols, :])
    return C


def csr_spmm_t(values: np.ndarray, B: np.ndarray, offsets, columns) -> np.ndarray:
    """C[h, col(k), :] += values[h, k] * B[h, row(k), :]  (transposed SpMM).

    cusparseSpMM with CUSPARSE_OPERATION_TRANSPOSE
    (models/block_attn.cu:526 dK = dS^T.Q, :536 dV = P^T.dO).
    Pinned by: dense matmul with the scattered matrix transposed (tests).
    """
    rows = csr_row_index(offsets)
    cols = np.asarray(columns, dtype=np.int64)
    NB, L, d = B.shape
    C = np.zeros((NB, L, d), dtype=values.dtype)
    np.add.at(C, (slice(None), cols), values[:, :, None] * B[:, rows, :])
    return C


def csr_softmax_scale_backward(dP: np.ndarray, P: np.ndarray, offsets, scale: float):
    """t = dP*P;  g_i = sum_row t;  dS = (t - P*g)*scale.

    models/block_attn.cu:90-130 (identical in block_attn_mask.cu:142-173).
    Returns (dS, t); the reference leaves ``t`` in the dP buffer.
    Pinned by: torch.autograd through ``dense_masked_attention`` and a float64
    finite-difference check on tiny shapes (tests).
    """
    rows = csr_row_index(offsets)
    t = dP * P
    g = np.zeros((P.shape[0], len(offsets) - 1), dtype=P.dtype)
    if P.shape[1]:
        np.add.at(g, (slice(None), rows), t)
    dS = (t - P * g[:, rows]) * P.dtype.type(scale)
    return dS, t


def csr_attention_forward(Q, K, V, offsets, columns, sum_mat, key_penalty=None):
    """Forward of models/block_attn.cu:453-487 (mask variant block_attn_mask.cu:530-596).

    Q, K, V: [NB, L, d].  Returns (O [NB, L, d], P [NB, n]).
    """
    NB, L, d = Q.shape
    scale = np.float32(1.0) / np.sqrt(np.float32(d))  # models/block_attn.cu:420 (fp32 sqrtf)
    S = csr_sddmm(Q, K, offsets, columns)
    P = csr_scale_softmax(S, offsets, sum_mat, L, scale, key_penalty, columns)
    O = csr_spmm(P, V, offsets, columns)
    return O, P


def csr_attention_backward(Q, K, V, P, dO, offsets, columns):
    """Backward of models/block_attn.cu:489-544.  Returns (dQ, dK, dV, dS)."""
    d = Q.shape[-1]
    scale = np.float32(1.0) / np.sqrt(np.float32(d))
    dP = csr_sddmm(dO, V, offsets, columns)
    dS, _ = csr_softmax_scale_backward(dP, P, offsets, scale)
    dQ = csr_spmm(dS, K, offsets, columns)
    dK = csr_spmm_t(dS, Q, offsets, columns)
    dV = csr_spmm_t(P, dO, offsets, columns)
    return dQ, dK, dV, dS


def key_penalty_from_mask(mask: np.ndarray, num_heads: int) -> np.ndarray:
    """[B, L] 0/1 key mask -> additive penalty [B*H, L] with flat index (b*H+h)*L + col.

    models/attention_blockcuda_mask.py:42-43: ``mask.repeat(1, H)`` then
    ``1e6 * (1 - mask)``.
    """
    mask = np.asarray(mask, dtype=np.float32)
    B, L = mask.shape
    rep = np.tile(mask, (1, num_heads)).reshape(B * num_heads, L)
    return (np.float32(1e6) * (np.float32(1.0) - rep)).astype(np.float32)


# --------------------------------------------------------------------------
# Dense formulation (torch, autograd) -- second statement + CPU baseline
# --------------------------------------------------------------------------
def dense_masked_attention(q, k, v, pattern, key_mask=None):
    """Dense PyTorch statement of the sparse semantics; differentiable.

    q, k, v: torch tensors [B, H, L, d]; ``pattern``: [L, L] 0/1 tensor;
    ``key_mask``: optional [B, L] 0/1.  Returns (O [B,H,L,d], P [B,H,L,L]).

        S = (q k^T)/sqrt(d);  S -= 1e6 (1-key_mask)   (mask variants only)
        S = S * pattern       (off-pattern logits become 0, NOT -inf;
                               models/block_attn.cu:70-72: (L-n_i) exp(-m))
        P = softmax(S) * pattern;  O = P v
    """
    import torch

    d = q.shape[-1]
    s = torch.matmul(q, k.transpose(-2, -1)) * float(np.float32(1.0) / np.sqrt(np.float32(d)))
    if key_mask is not None:
        s = s - 1e6 * (1.0 - key_mask.to(s.dtype))[:, None, None, :]
    m = pattern.to(s.dtype)
    s = s * m
    p = torch.softmax(s, dim=-1) * m
    return torch.matmul(p, v), p
