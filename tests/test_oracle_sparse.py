"""Pins for oracle/sparse_attention.py and oracle/dense_attention.py (CPU only).

The reference holds no golden vectors for this path, so every oracle function
is pinned by mathematics: brute force on tiny inputs, special cases that reduce
to library routines, invariants, finite differences and a second independent
formulation (dense PyTorch + autograd).
"""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from oracle import dense_attention as oda


def _rand_block_mask(nb, rng, p=0.3):
    mat = (rng.random((nb, nb)) < p).astype(np.float32)
    mat[np.arange(nb), np.arange(nb)] = 1
    return mat


def _scatter(values, offsets, columns, L):
    rows = osa.csr_row_index(offsets)
    M = np.zeros((values.shape[0], L, L), dtype=values.dtype)
    M[:, rows, columns] = values
    return M


# ------------------------------------------------------------------ CSR builder
@pytest.mark.parametrize("nb,bs", [(4, 2), (5, 3), (8, 4), (3, 1)])
def test_block_csr_matches_brute_force(nb, bs):
    rng = np.random.default_rng(nb * 10 + bs)
    mat = _rand_block_mask(nb, rng)
    mat[1, :] = 0  # an empty block row
    sum_mat, offsets, columns = osa.build_csr_from_block_mask(mat, bs)
    L = nb * bs
    exp_cols, exp_sum = [], []
    for i in range(L):
        row = [j for j in range(L) if mat[i // bs, j // bs] != 0]
        exp_cols += row
        exp_sum.append(len(row))
    assert sum_mat.tolist() == exp_sum
    assert offsets.tolist() == [0] + np.cumsum(exp_sum).tolist()
    assert columns.tolist() == exp_cols
    assert offsets[-1] == bs * bs * int(mat.sum())
    assert sum_mat.dtype == np.int32 and offsets.dtype == np.int32 and columns.dtype == np.int32


def test_element_csr_is_block_csr_with_bs1():
    rng = np.random.default_rng(3)
    pat = (rng.random((12, 12)) < 0.4).astype(np.float32)
    a = osa.csr_from_dense_pattern(pat)
    b = osa.build_csr_from_block_mask(pat, 1)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


# ------------------------------------------------------------------ SDDMM / SpMM
def test_sddmm_and_spmm_match_dense_and_loops():
    rng = np.random.default_rng(0)
    nb, bs, d, NB = 4, 4, 8, 3
    L = nb * bs
    mat = _rand_block_mask(nb, rng)
    sum_mat, offsets, columns = osa.build_csr_from_block_mask(mat, bs)
    Q, K, V = (rng.standard_normal((NB, L, d)) for _ in range(3))
    S = osa.csr_sddmm(Q, K, offsets, columns)
    # brute force triple loop
    k = 0
    for i in range(L):
        for kk in range(offsets[i], offsets[i + 1]):
            j = columns[kk]
            for h in range(NB):
                acc = 0.0
                for t in range(d):
                    acc += Q[h, i, t] * K[h, j, t]
                assert abs(S[h, kk] - acc) < 1e-12
            k += 1
    assert k == len(columns)
    dense = _scatter(S, offsets, columns, L)
    pat = np.repeat(np.repeat(mat, bs, 0), bs, 1)
    assert np.allclose(dense, np.einsum("hid,hjd->hij", Q, K) * pat, atol=1e-12)
    # SpMM N and T against dense products with the scattered matrix
    W = rng.standard_normal(S.shape)
    Wd = _scatter(W, offsets, columns, L)
    assert np.allclose(osa.csr_spmm(W, V, offsets, columns), Wd @ V, atol=1e-12)
    assert np.allclose(osa.csr_spmm_t(W, V, offsets, columns), Wd.transpose(0, 2, 1) @ V, atol=1e-12)


# ------------------------------------------------------------------ softmax
def test_softmax_full_pattern_is_ordinary_softmax():
    rng = np.random.default_rng(1)
    L, NB = 16, 2
    mat = np.ones((4, 4), dtype=np.float32)
    sum_mat, offsets, columns = osa.build_csr_from_block_mask(mat, 4)
    S = rng.standard_normal((NB, L * L)) * 3
    P = osa.csr_scale_softmax(S, offsets, sum_mat, L, 0.25)
    ref = torch.softmax(torch.from_numpy(S.reshape(NB, L, L) * 0.25), -1).numpy().reshape(NB, -1)
    assert np.allclose(P, ref, rtol=1e-13, atol=1e-15)


def test_softmax_row_sum_invariant_and_off_pattern_zero_logits():
    rng = np.random.default_rng(2)
    nb, bs, NB = 6, 4, 2
    L = nb * bs
    mat = _rand_block_mask(nb, rng)
    sum_mat, offsets, columns = osa.build_csr_from_block_mask(mat, bs)
    S = rng.standard_normal((NB, len(columns))) * 4
    scale = 0.3
    P = osa.csr_scale_softmax(S, offsets, sum_mat, L, scale)
    Pd = _scatter(P, offsets, columns, L)
    # independent statement: full-row softmax where off-pattern logits are exactly 0
    Sd = _scatter(S * scale, offsets, columns, L)
    full = np.exp(Sd) / np.exp(Sd).sum(-1, keepdims=True)
    pat = np.repeat(np.repeat(mat, bs, 0), bs, 1)
    assert np.allclose(Pd, full * pat, rtol=1e-12, atol=1e-15)
    # rows sum to 1 - (L-n_i)/sum_j exp(s_ij)
    expect = 1.0 - (L - sum_mat)[None] / np.exp(Sd).sum(-1)
    assert np.allclose(Pd.sum(-1), expect, rtol=1e-12)
    assert (Pd.sum(-1) < 1.0 + 1e-12).all()


def _serial_softmax_row(vals, cols, penalty_row, L, scale):
    """Scalar transcription of the recipe of the serial kernel
    models/block_attn_mask.cu:28-66 (max starts at -100 there)."""
    v = [float(x) * scale - (penalty_row[c] if penalty_row is not None else 0.0) for x, c in zip(vals, cols)]
    m = -100.0
    for x in v:
        if m < x:
            m = x
    s = 0.0
    for x in v:
        s += np.exp(x - m)
    s += (L - len(v)) * np.exp(-m)
    r = 1.0 / s
    return [0.0 if r == 0 else np.exp(x - m) * r for x in v]


@pytest.mark.parametrize("with_mask", [False, True])
def test_softmax_matches_serial_recipe(with_mask):
    rng = np.random.default_rng(5)
    L, NB = 12, 2
    pat = (rng.random((L, L)) < 0.4)
    pat[3, :] = False  # empty row
    sum_mat, offsets, columns = osa.csr_from_dense_pattern(pat)
    S = rng.standard_normal((NB, len(columns))) * 5
    pen = None
    if with_mask:
        km = np.ones((NB, L), dtype=np.float32)
        km[0, 8:] = 0
        km[1, 5:] = 0
        pen = osa.key_penalty_from_mask(km, 1).astype(np.float64)
    P = osa.csr_scale_softmax(S, offsets, sum_mat, L, 0.4, pen, columns)
    for h in range(NB):
        for i in range(L):
            a, b = offsets[i], offsets[i + 1]
            exp = _serial_softmax_row(S[h, a:b], columns[a:b], None if pen is None else pen[h], L, 0.4)
            # max initialiser differs between variants (-100 / 0): shift invariance
            assert np.allclose(P[h, a:b], exp, rtol=1e-12, atol=1e-300)
    if with_mask:
        Pd = _scatter(P, offsets, columns, L)
        assert (Pd[0, :, 8:] == 0).all() and (Pd[1, :, 5:] == 0).all()  # exact zeros on padded keys


def test_softmax_overflow_guard_gives_zero_in_fp32():
    # every logit far below -88.7: (L-n)*expf(-m) overflows fp32 -> r == 0 -> P = 0
    pat = np.zeros((4, 4), dtype=bool)
    pat[:, 0] = True
    sum_mat, offsets, columns = osa.csr_from_dense_pattern(pat)
    S = np.full((1, 4), -95.0, dtype=np.float32)
    P = osa.csr_scale_softmax(S, offsets, sum_mat, 4, 1.0)
    assert (P == 0).all()


def test_key_penalty_layout():
    mask = np.array([[1, 1, 0], [1, 0, 0]], dtype=np.float32)
    pen = osa.key_penalty_from_mask(mask, 2)
    assert pen.shape == (4, 3)
    assert np.array_equal(pen[0], pen[1]) and np.array_equal(pen[2], pen[3])
    assert pen[0].tolist() == [0, 0, 1e6] and pen[2].tolist() == [0, 1e6, 1e6]


# ------------------------------------------------------------------ whole fwd/bwd vs dense autograd
@pytest.mark.parametrize("with_mask", [False, True])
def test_csr_pipeline_matches_dense_autograd(with_mask):
    rng = np.random.default_rng(7)
    B, H, nb, bs, d = 2, 2, 4, 4, 8
    L = nb * bs
    mat = _rand_block_mask(nb, rng)
    sum_mat, offsets, columns = osa.build_csr_from_block_mask(mat, bs)
    q, k, v, do = (torch.from_numpy(rng.standard_normal((B, H, L, d))) for _ in range(4))
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    key_mask = None
    pen = None
    if with_mask:
        km = np.ones((B, L), dtype=np.float32)
        km[0, 10:] = 0
        km[1, 13:] = 0
        key_mask = torch.from_numpy(km)
        pen = osa.key_penalty_from_mask(km, H).astype(np.float64)
    pat = torch.from_numpy(np.repeat(np.repeat(mat, bs, 0), bs, 1))
    O, P = osa.dense_masked_attention(q, k, v, pat, key_mask)
    O.backward(do)
    f = lambda t: t.detach().numpy().reshape(B * H, L, -1)
    Oc, Pc = osa.csr_attention_forward(f(q), f(k), f(v), offsets, columns, sum_mat, pen)
    assert np.allclose(Oc, f(O), rtol=1e-10, atol=1e-12)
    assert np.allclose(_scatter(Pc, offsets, columns, L), f(P), rtol=1e-10, atol=1e-14)
    dQ, dK, dV, _ = osa.csr_attention_backward(f(q), f(k), f(v), Pc, f(do), offsets, columns)
    assert np.allclose(dQ, f(q.grad), rtol=1e-9, atol=1e-11)
    assert np.allclose(dK, f(k.grad), rtol=1e-9, atol=1e-11)
    assert np.allclose(dV, f(v.grad), rtol=1e-9, atol=1e-11)


def test_backward_finite_differences():
    rng = np.random.default_rng(11)
    NB, L, d = 1, 6, 3
    pat = rng.random((L, L)) < 0.5
    pat[np.arange(L), np.arange(L)] = True
    sum_mat, offsets, columns = osa.csr_from_dense_pattern(pat)
    Q, K, V, dO = (rng.standard_normal((NB, L, d)) for _ in range(4))
    _, P = osa.csr_attention_forward(Q, K, V, offsets, columns, sum_mat)
    dQ, dK, dV, _ = osa.csr_attention_backward(Q, K, V, P, dO, offsets, columns)

    def loss(q, k, v):
        return float((osa.csr_attention_forward(q, k, v, offsets, columns, sum_mat)[0] * dO).sum())

    eps = 1e-6
    for X, G, idx in ((Q, dQ, 0), (K, dK, 1), (V, dV, 2)):
        for pos in [(0, 1, 2), (0, 4, 0), (0, 5, 1)]:
            args = [Q.copy(), K.copy(), V.copy()]
            args[idx][pos] += eps
            up = loss(*args)
            args[idx][pos] -= 2 * eps
            dn = loss(*args)
            assert abs((up - dn) / (2 * eps) - G[pos]) < 1e-6


# ------------------------------------------------------------------ dense phase
@pytest.mark.parametrize("with_mask", [False, True])
def test_dense_attention_matches_torch(with_mask):
    rng = np.random.default_rng(13)
    NB, L, d = 3, 10, 4
    Q, K, V, dO = (rng.standard_normal((NB, L, d)) for _ in range(4))
    pen = None
    bias = None
    if with_mask:
        km = np.ones((NB, L), dtype=np.float32)
        km[:, 7:] = 0
        pen = osa.key_penalty_from_mask(km, 1).astype(np.float64)
        bias = torch.from_numpy(-pen)[:, None, :]
    O, P = oda.dense_attention_forward(Q, K, V, pen)
    q, k, v = (torch.from_numpy(x).requires_grad_() for x in (Q, K, V))
    scale = float(np.float32(1.0) / np.sqrt(np.float32(d)))
    s = q @ k.transpose(-1, -2) * scale
    if bias is not None:
        s = s + bias
    p = torch.softmax(s, -1)
    o = p @ v
    o.backward(torch.from_numpy(dO))
    assert np.allclose(O, o.detach().numpy(), rtol=1e-10, atol=1e-12)
    assert np.allclose(P, p.detach().numpy(), rtol=1e-10, atol=1e-14)
    dQ, dK, dV = oda.dense_attention_backward(Q, K, V, P, dO)
    assert np.allclose(dQ, q.grad.numpy(), rtol=1e-9, atol=1e-11)
    assert np.allclose(dK, k.grad.numpy(), rtol=1e-9, atol=1e-11)
    assert np.allclose(dV, v.grad.numpy(), rtol=1e-9, atol=1e-11)
    if not with_mask:
        ref = torch.nn.functional.scaled_dot_product_attention(
            torch.from_numpy(Q), torch.from_numpy(K), torch.from_numpy(V), scale=scale
        )
        assert np.allclose(O, ref.numpy(), rtol=1e-9, atol=1e-11)
