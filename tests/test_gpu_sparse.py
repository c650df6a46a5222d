"""Parity of the sparse-attention HIP kernels with the float64 oracle, through the C ABI (GPU box only).

Tolerance: fp32 results within 1e-4 relative (see abi_utils.assert_close).
"""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from spion_amd import workloads
from tests.abi_utils import SparseABI, assert_close, oracle_fwd_bwd, run_and_check

pytestmark = pytest.mark.gpu


def _inputs(NB, L, d, seed, scale=1.0, dev="cuda"):
    g = torch.Generator().manual_seed(seed)
    return tuple((torch.randn(NB, L, d, generator=g) * s).to(dev) for s in (scale, scale, 1.0, 1.0))


def _random_block_mask(nb, p, seed, empty_row=None, empty_col=None):
    rng = np.random.default_rng(seed)
    mat = (rng.random((nb, nb)) < p).astype(np.float32)
    mat[np.arange(nb), np.arange(nb)] = 1
    if empty_row is not None:
        mat[empty_row, :] = 0
    if empty_col is not None:
        mat[:, empty_col] = 0
    return mat


# ---------------------------------------------------------------------------------- tile (MFMA) path
@pytest.mark.parametrize(
    "L,bs,d,NB,p",
    [
        (128, 32, 32, 3, 0.15),   # about one tile per strip  -> 1 wavefront per strip
        (256, 32, 32, 2, 0.30),   # 2-3 tiles per strip       -> 2 wavefronts
        (256, 32, 32, 5, 0.80),   # many tiles                -> 4 wavefronts
        (256, 64, 32, 2, 0.40),   # 64x64 blocks = 2x2 tiles
        (256, 32, 64, 2, 0.50),   # head dim 64
        (512, 128, 64, 1, 0.50),
        # launches of 2048 block rows and more take the fewest wavefronts that keep a row's logits in registers
        (256, 32, 32, 256, 0.50),   # 2048 rows of at most 8 tiles  -> 1 wavefront, register-resident
        (512, 32, 32, 128, 0.60),   # 2048 rows of up to 16 tiles   -> 2 wavefronts
        (256, 32, 32, 160, 0.50),   # 1280 rows                     -> at least 2 wavefronts
        (256, 32, 64, 256, 0.40),   # head dim 64: 4 tiles per wavefront
    ],
)
def test_tile_path_matches_oracle(L, bs, d, NB, p):
    nb = L // bs
    mat = _random_block_mask(nb, p, seed=L + bs + d)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=1, scale=1.5)
    run_and_check(abi, Q, K, V, dO, tag=f"tile L={L} bs={bs} d={d}")
    assert abi.last_path() == 1
    abi.close()


def test_tile_path_empty_block_row_and_column():
    L, bs, d, NB = 256, 32, 32, 2
    mat = _random_block_mask(L // bs, 0.4, seed=5, empty_row=2, empty_col=5)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=2)
    got, _ = run_and_check(abi, Q, K, V, dO, tag="empty strip")
    assert (got["O"][:, 64:96] == 0).all() and (got["dQ"][:, 64:96] == 0).all()
    assert (got["dK"][:, 160:192] == 0).all() and (got["dV"][:, 160:192] == 0).all()
    abi.close()


def test_tile_path_full_pattern_is_softmax_attention():
    L, bs, d, NB = 128, 32, 32, 2
    sm, off, col = osa.build_csr_from_block_mask(np.ones((4, 4), np.float32), bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=3)
    O, P = abi.forward(Q, K, V)
    ref = torch.nn.functional.scaled_dot_product_attention(Q.double().cpu(), K.double().cpu(), V.double().cpu())
    assert_close(O.cpu().numpy(), ref.numpy(), what="full pattern O")
    assert_close(P.view(NB, L, L).sum(-1).cpu().numpy(), np.ones((NB, L)), what="row sums")
    abi.close()


@pytest.mark.parametrize("d", [32, 64])
def test_tile_path_with_key_mask(d):
    L, bs, B, H = 256, 32, 3, 2
    NB = B * H
    mat = _random_block_mask(L // bs, 0.35, seed=8)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    key_mask = np.ones((B, L), np.float32)
    key_mask[0, 200:] = 0
    key_mask[1, 77:] = 0       # not tile aligned
    pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask, H)).cuda()
    abi = SparseABI(d, L, NB, bs, with_mask=True)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=4)
    got, _ = run_and_check(abi, Q, K, V, dO, penalty=pen, tag="key mask")
    # probabilities of padded keys are exactly zero
    rows = osa.csr_row_index(off)
    padded = torch.from_numpy(col.astype(np.int64) >= 77).cuda()
    assert (got["P"][2][padded] == 0).all() and (got["P"][3][padded] == 0).all()
    abi.close()


@pytest.mark.parametrize("L,d,with_mask", [(2048, 32, False), (2048, 32, True), (1024, 64, False), (1024, 64, True),
                                           (2048, 64, False), (2048, 64, True)])
def test_tile_path_global_row_and_column(L, d, with_mask):
    """A block row and a block column that span the whole sequence: rows too long for the register-resident
    forward (two-sweep kernel), long strips walked by several wavefronts in the backward passes, and the
    one-pass backward without the kept copy of O.  At L = 2048 the global strips count as long against the rest
    (more than 32 tiles): every pass is then two launches -- the long strips with eight wavefronts each on the
    caller's stream, the others on the handle's side stream."""
    from spion_amd import _lib
    bs, B, H = 32, 1, 2
    NB, nb = B * H, L // bs
    mat = _random_block_mask(nb, 0.04, seed=L + d)
    mat[0, :] = 1
    mat[:, 0] = 1
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=12, scale=1.3)
    pen = None
    if with_mask:
        key_mask = np.ones((B, L), np.float32)
        key_mask[0, L - 301:] = 0
        pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask, H)).cuda()
    got, ref = run_and_check(abi, Q, K, V, dO, penalty=pen, tag=f"global row/column L={L} d={d}")
    assert abi.last_path() == 1
    _lib.core().spion_use_output_cache(abi.handle, 0)  # backward must find g by its own sweep now
    dQ, dK, dV = abi.backward(Q, K, V, got["P"], dO)
    for name, t in (("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(t.cpu().numpy(), ref[name], what=f"global row/column, no O copy: {name}")
    abi.close()


@pytest.mark.parametrize("d", [32, 64])
def test_tile_path_global_strips_beside_one_wavefront_strips(d):
    """Many heads (2560 strips a launch): the strips other than the global ones take one wavefront each in the
    backward passes -- the launch on the side stream -- while the global row and column take eight."""
    L, bs, NB = 2048, 32, 40
    nb = L // bs
    mat = _random_block_mask(nb, 0.05, seed=77 + d)
    mat[3, :] = 1
    mat[:, 5] = 1
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=31, scale=1.1)
    run_and_check(abi, Q, K, V, dO, tag=f"global strips, NB={NB}, d={d}")
    assert abi.last_path() == 1
    abi.close()


@pytest.mark.parametrize("with_mask", [False, True])
def test_tile_path_d64_mixed_strip_lengths_in_one_forward_launch(with_mask):
    """Head dimension 64, four wavefronts per strip, most strips of 12 to 23 tiles and one global block row of 64: the
    forward keeps six logit tiles per wavefront in registers and the global row takes the two sweeps inside the same
    launch (models/block_attn.cu:33-130 makes no such distinction; the results must not show it)."""
    L, d, bs, B, H = 2048, 64, 32, 1, 2
    NB, nb = B * H, L // bs
    mat = workloads.band_random_block_mask(nb, 8, extra_frac=0.05, seed=9)
    mat[0, :] = 1
    rows = mat.sum(1)
    assert rows.max() == nb and np.sort(rows)[-2] <= 24 and np.median(rows) > 16
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=21, scale=1.2)
    pen = None
    if with_mask:
        key_mask = np.ones((B, L), np.float32)
        key_mask[0, L - 200:] = 0
        pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask, H)).cuda()
    run_and_check(abi, Q, K, V, dO, penalty=pen, tag=f"d=64 mixed strip lengths mask={with_mask}")
    assert abi.last_path() == 1
    abi.close()


def test_row_sum_invariant_large_logits_and_guard():
    # logits of +-30: exp range exercised; every row still obeys sum P = 1 - (L-n) e^{-m} / Z
    L, bs, d, NB = 128, 32, 32, 2
    mat = _random_block_mask(4, 0.5, seed=9)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=6, scale=3.0)
    run_and_check(abi, Q, K, V, dO, tag="large logits")
    # every logit below -88.7 -> denominator overflows in fp32 -> P == 0 exactly (reference guard)
    Q2 = torch.full_like(Q, 8.0)
    K2 = torch.full_like(K, -8.0)          # q.k/sqrt(32) = -362
    O, P = abi.forward(Q2, K2, V)
    sparse_rows = torch.from_numpy(np.repeat(sm < L, sm)).cuda()
    assert (P[:, sparse_rows] == 0).all()
    abi.close()


# ---------------------------------------------------------------------------------- element path
def _random_element_csr(L, p, seed, empty_row=None):
    rng = np.random.default_rng(seed)
    pat = rng.random((L, L)) < p
    pat[np.arange(L), np.arange(L)] = True
    if empty_row is not None:
        pat[empty_row, :] = False
    return osa.csr_from_dense_pattern(pat)


@pytest.mark.parametrize("L,d,NB,p", [(96, 32, 3, 0.2), (100, 16, 2, 0.5), (160, 64, 2, 0.9), (70, 128, 2, 0.3)])
def test_element_path_matches_oracle(L, d, NB, p):
    sm, off, col = _random_element_csr(L, p, seed=L + d, empty_row=7)
    abi = SparseABI(d, L, NB, 1, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=10, scale=1.2)
    got, _ = run_and_check(abi, Q, K, V, dO, tag=f"element L={L} d={d}")
    assert abi.last_path() == (3 if d == 32 and L % 32 == 0 else 2)   # 3: hybrid (dense tiles + gathers)
    assert (got["O"][:, 7] == 0).all() and (got["dQ"][:, 7] == 0).all()
    abi.close()


def test_element_path_with_key_mask():
    L, d, B, H = 192, 32, 2, 2
    sm, off, col = _random_element_csr(L, 0.25, seed=21)
    key_mask = np.ones((B, L), np.float32)
    key_mask[0, 150:] = 0
    key_mask[1, 31:] = 0
    pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask, H)).cuda()
    abi = SparseABI(d, L, B * H, 1, with_mask=True)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(B * H, L, d, seed=11)
    run_and_check(abi, Q, K, V, dO, penalty=pen, tag="element key mask")
    abi.close()


def test_tile_and_element_paths_agree():
    """Two independent kernel families on the same block pattern."""
    L, bs, d, NB = 512, 32, 32, 4
    mat = _random_block_mask(L // bs, 0.2, seed=31)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    Q, K, V, dO = _inputs(NB, L, d, seed=12)
    res = []
    for force in (False, True):
        abi = SparseABI(d, L, NB, bs, with_mask=False)
        abi.force_element(force)
        abi.set_pattern(sm, off, col)
        O, P = abi.forward(Q, K, V)
        dQ, dK, dV = abi.backward(Q, K, V, P, dO)
        assert abi.last_path() == (2 if force else 1)
        res.append([t.cpu().numpy() for t in (O, P, dQ, dK, dV)])
        abi.close()
    for a, b, name in zip(res[0], res[1], ["O", "P", "dQ", "dK", "dV"]):
        assert_close(a, b, what=f"tile vs element {name}")


@pytest.mark.parametrize("with_mask", [False, True])
def test_hybrid_and_gather_paths_agree(with_mask):
    """A window + random-columns pattern (benchmark configuration 4 in small): the hybrid kernels (window tiles on
    the MFMA units with bit masks, the rest gathered) against the pure gather kernels and the oracle; every way the
    backward can get its row sums (the caller's Out, the handle's kept copy, neither -> gather kernels)."""
    from spion_amd import _lib

    L, d, NB = 512, 32, 3
    sm, off, col = workloads.window_random_csr(L, 48, 150, seed=9)
    Q, K, V, dO = _inputs(NB, L, d, seed=14)
    pen = None
    if with_mask:
        valid = torch.tensor([L, 300, 77])
        pen = (1e6 * (torch.arange(L)[None, :] >= valid[:, None]).float()).cuda().contiguous()
    ref = oracle_fwd_bwd(Q, K, V, dO, sm, off, col, penalty=pen)
    res = {}
    for force in (False, True):
        abi = SparseABI(d, L, NB, 1, with_mask=with_mask)
        abi.force_element(force)
        abi.set_pattern(sm, off, col)
        O, P = abi.forward(Q, K, V, pen)
        assert abi.last_path() == (2 if force else 3)
        grads = {"abi": abi.backward(Q, K, V, P, dO)}                       # kept copy of Out (hybrid) / gathers
        assert abi.last_path() == (2 if force else 3)
        grads["with_out"] = abi.backward_rowmajor(Q, K, V, P, O, dO)        # the caller hands Out over
        if not force:
            _lib.core().spion_use_output_cache(abi.handle, 0)
            O2, P2 = abi.forward(Q, K, V, pen)
            assert torch.equal(O2, O) and torch.equal(P2, P)
            grads["no_out"] = abi.backward(Q, K, V, P2, dO)                  # nothing to take row sums from
            assert abi.last_path() == 2
        for how, g in grads.items():
            for name, t in zip(("dQ", "dK", "dV"), g):
                assert_close(t.cpu().numpy(), ref[name], what=f"force={force} {how} {name}")
        assert_close(O.cpu().numpy(), ref["O"], what=f"force={force} O")
        assert_close(P.cpu().numpy(), ref["P"], what=f"force={force} P")
        if with_mask:
            cols = torch.from_numpy(col.astype(np.int64)).cuda()
            assert (P[pen[:, cols] > 0] == 0).all()
        res[force] = (O, P) + grads["abi"]
        abi.close()
    for a, b, name in zip(res[False], res[True], ["O", "P", "dQ", "dK", "dV"]):
        assert_close(a.cpu().numpy(), b.cpu().numpy(), what=f"hybrid vs gather {name}")


@pytest.mark.parametrize("L,NB", [(1024, 256), (2048, 64), (1024, 64)])
def test_hybrid_remainder_columns_from_lds_on_many_heads(L, NB):
    """With enough heads for 256 work-groups of 1024, 512 or 256 columns (the three cases), the column pass of the
    remainder (hybrid kernels) and of all entries (element kernels) keeps the Q and dO rows of a range of 512 rows in
    LDS (two and four ranges here):
    the two families against each other on all heads, three heads against the oracle; a second backward and the
    strided entry points give the same bits."""
    d = 32
    sm, off, col = workloads.window_random_csr(L, 48, 110, seed=L)
    Q, K, V, dO = _inputs(NB, L, d, seed=L + 1)
    res = {}
    for force in (False, True):
        abi = SparseABI(d, L, NB, 1, with_mask=False)
        abi.force_element(force)
        abi.set_pattern(sm, off, col)
        O, P = abi.forward(Q, K, V, None)
        assert abi.last_path() == (2 if force else 3)
        res[force] = (O, P) + tuple(abi.backward_rowmajor(Q, K, V, P, O, dO))
        again = abi.backward_rowmajor(Q, K, V, P, O, dO)
        for x, y in zip(res[force][2:], again):
            assert torch.equal(x, y)
        # the same heads as views of [B, L, H*d] projections: bit for bit
        H = 2
        B = NB // H
        proj = lambda t: t.view(B, H, L, d).transpose(1, 2).contiguous().transpose(1, 2)
        q, k, v, do = (proj(t) for t in (Q, K, V, dO))
        out, dq, dk, dv = (proj(torch.full_like(Q, float("nan"))) for _ in range(4))
        assert not q.is_contiguous()
        Ps = abi.forward_strided(q, k, v, out)
        abi.backward_strided(q, k, v, Ps, out, do, dq, dk, dv)
        assert abi.last_path() == (2 if force else 3)
        for x, y in zip((out, Ps, dq, dk, dv), res[force]):
            assert torch.equal(x.reshape(y.shape), y)
        abi.close()
    for a, b, name in zip(res[False], res[True], ["O", "P", "dQ", "dK", "dV"]):
        assert_close(a.cpu().numpy(), b.cpu().numpy(), what=f"hybrid vs gather {name}")
    for h in (0, NB // 2 + 13, NB - 1):
        ref = oracle_fwd_bwd(Q[h:h + 1], K[h:h + 1], V[h:h + 1], dO[h:h + 1], sm, off, col)
        for t, name in zip(res[False], ["O", "P", "dQ", "dK", "dV"]):
            assert_close(t[h:h + 1].cpu().numpy(), ref[name], what=f"head {h} {name}")


def test_hybrid_pattern_with_partial_tiles_empty_rows_and_no_remainder():
    """Dense tiles with holes, rows without any entry and a block row whose entries all sit in dense tiles."""
    L, d, NB = 256, 32, 2
    rng = np.random.default_rng(5)
    keep = np.zeros((L, L), bool)
    for I in range(L // 32):
        for J in (I, (I + 3) % (L // 32)):
            keep[I * 32:(I + 1) * 32, J * 32:(J + 1) * 32] = rng.random((32, 32)) < 0.6   # two half-filled tiles
    keep[64:96] = False
    keep[64:96, 64:96] = True                       # block row 2: one full tile, nothing else
    extra = rng.random((L, L)) < 0.02               # a few scattered entries elsewhere
    extra[64:96] = False
    keep |= extra
    keep[5] = False                                 # empty rows
    keep[200] = False
    sm = keep.sum(1).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(sm)]).astype(np.int32)
    col = np.nonzero(keep)[1].astype(np.int32)
    abi = SparseABI(d, L, NB, 1, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=15, scale=1.3)
    got, _ = run_and_check(abi, Q, K, V, dO, tag="hybrid partial tiles")
    assert abi.last_path() == 3
    assert (got["O"][:, 5] == 0).all() and (got["dQ"][:, 200] == 0).all()
    abi.close()


# ---------------------------------------------------------------------------------- benchmark configurations
def test_config1_block_sparse_l1024():
    """B=8, H=2, L=1024, d=32, 32x32 blocks, band of 3 + 5 % random blocks; inputs N(0,1)/sqrt(32)."""
    B, H, L, d, bs = 8, 2, 1024, 32, 32
    mat = workloads.config1_mask()
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    q, k, v, do = workloads.qkv(B, H, L, d, scale=1.0 / np.sqrt(32.0), seed=0, device="cuda")
    abi = SparseABI(d, L, B * H, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    f = lambda t: t.reshape(B * H, L, d).contiguous()
    run_and_check(abi, f(q), f(k), f(v), f(do), tag="config 1")
    assert abi.last_path() == 1
    abi.close()


def test_config4_element_sparse_small_heads():
    """Config 4 shape (L=4096, d=32, window +-64 plus random columns to 5 %, key padding) on 2x2 heads."""
    B, H, L, d = 2, 2, 4096, 32
    sm, off, col = workloads.window_random_csr(L, 64, 205, seed=3)
    key_mask = workloads.valid_length_mask(B, L, 2048, 4096, seed=5)
    pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask.numpy(), H)).cuda()
    q, k, v, do = workloads.qkv(B, H, L, d, seed=0, device="cuda")
    abi = SparseABI(d, L, B * H, 1, with_mask=True)
    abi.set_pattern(sm, off, col)
    f = lambda t: t.reshape(B * H, L, d).contiguous()
    run_and_check(abi, f(q), f(k), f(v), f(do), penalty=pen, tag="config 4")
    assert abi.last_path() == 3
    abi.close()


def test_north_star_shape_properties():
    """L=4096, H=2, d=32, 10 % block density at the benchmark batch: size-independent checks
    (row-sum invariant, linearity of the backward in dO, tile path == element path on one head pair)
    plus the oracle on two of the 64 heads."""
    B, H, L, d, bs = 32, 2, 4096, 32, 32
    NB = B * H
    mat = workloads.north_star_mask(bs)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    q, k, v, do = workloads.qkv(B, H, L, d, seed=0, device="cuda")
    f = lambda t: t.reshape(NB, L, d).contiguous()
    Q, K, V, dO = f(q), f(k), f(v), f(do)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    O, P = abi.forward(Q, K, V)
    dQ, dK, dV = abi.backward(Q, K, V, P, dO)
    assert abi.last_path() == 1
    # (a) oracle on heads 0 and 63
    from tests.abi_utils import oracle_fwd_bwd
    for hsel in (0, NB - 1):
        s = slice(hsel, hsel + 1)
        ref = oracle_fwd_bwd(Q[s], K[s], V[s], dO[s], sm, off, col)
        for name, got in (("O", O), ("P", P), ("dQ", dQ), ("dK", dK), ("dV", dV)):
            assert_close(got[s].cpu().numpy(), ref[name], what=f"north star head {hsel} {name}")
    # (b) rows of P sum to less than one and are non-negative; all finite
    rows = torch.from_numpy(osa.csr_row_index(off)).cuda()
    rs = torch.zeros(NB, L, device="cuda").index_add_(1, rows, P)
    assert torch.isfinite(P).all() and (P >= 0).all() and (rs <= 1 + 1e-5).all() and (rs > 0).all()
    # (c) the backward is linear in dO
    dQ2, dK2, dV2 = abi.backward(Q, K, V, P, 2.0 * dO)
    for a, b in ((dQ, dQ2), (dK, dK2), (dV, dV2)):
        assert torch.allclose(2.0 * a, b, rtol=1e-5, atol=1e-5)
    abi.close()
    # (d) element path on the first 4 heads agrees with the tile path
    abi2 = SparseABI(d, L, 4, bs, with_mask=False)
    abi2.force_element(True)
    abi2.set_pattern(sm, off, col)
    O2, P2 = abi2.forward(Q[:4], K[:4], V[:4])
    e = abi2.backward(Q[:4], K[:4], V[:4], P2, dO[:4])
    assert abi2.last_path() == 2
    for a, b, name in ((O[:4], O2, "O"), (P[:4], P2, "P"), (dQ[:4], e[0], "dQ"), (dK[:4], e[1], "dK"), (dV[:4], e[2], "dV")):
        assert_close(a.cpu().numpy(), b.cpu().numpy(), what=f"north star tile vs element {name}")
    abi2.close()


# ---------------------------------------------------------------------------------- module level (autograd)
@pytest.mark.parametrize("with_mask", [False, True])
def test_block_modules_autograd_match_dense_statement(with_mask):
    import spion_amd

    B, H, L, d, bs = 2, 2, 256, 32, 32
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    mat_np = _random_block_mask(L // bs, 0.3, seed=41)
    mat = torch.from_numpy(mat_np).cuda()
    if with_mask:
        cpp = spion_amd.Attention._blockcuda_mask_compile_module()
        mod = spion_amd.CUDABlockMaskAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    else:
        cpp = spion_amd.Attention._blockcuda_compile_module()
        mod = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    q, k, v, do = workloads.qkv(B, H, L, d, seed=3, device="cuda")
    key_mask = torch.ones(B, L)
    if with_mask:
        key_mask[0, 100:] = 0
    for t in (q, k, v):
        t.requires_grad_()
    for it in range(2):  # second call goes through the CSR cache
        out, attn = mod(q, k, v, key_mask.cuda(), mat)
        out.backward(do)
    if with_mask:
        assert attn == 0
    else:
        assert attn.shape == (B * H * int(mat_np.sum()) * bs * bs,)
    qc, kc, vc = (t.detach().double().cpu().requires_grad_() for t in (q, k, v))
    pat = torch.from_numpy(np.repeat(np.repeat(mat_np, bs, 0), bs, 1)).double()
    O, _ = osa.dense_masked_attention(qc, kc, vc, pat, key_mask.double() if with_mask else None)
    O.backward(do.double().cpu())
    assert_close(out.detach().cpu().numpy(), O.detach().numpy(), what="module out")
    for name, a, b in (("dq", q, qc), ("dk", k, kc), ("dv", v, vc)):
        assert_close(a.grad.cpu().numpy() / 2.0, b.grad.numpy(), what=f"module {name}")  # two backward passes accumulated


@pytest.mark.parametrize("with_mask", [False, True])
def test_block_modules_read_projection_views_in_place(with_mask):
    """Heads handed over as views of [B, L, H*d] projections (what models/attention.py:136-139 makes): the module
    takes them without copies, returns ``out`` in the same interleaved memory, and every result equals, bit for bit,
    what it returns for contiguous copies of the same tensors."""
    import spion_amd

    B, H, L, d, bs = 2, 2, 256, 32, 32
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    mat_np = _random_block_mask(L // bs, 0.3, seed=5)
    mat = torch.from_numpy(mat_np).cuda()
    if with_mask:
        cpp = spion_amd.Attention._blockcuda_mask_compile_module()
        mod = spion_amd.CUDABlockMaskAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    else:
        cpp = spion_amd.Attention._blockcuda_compile_module()
        mod = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    assert mod.reads_views
    g = torch.Generator().manual_seed(11)
    proj = [torch.randn(B, L, H * d, generator=g).cuda().requires_grad_() for _ in range(3)]
    dmerged = torch.randn(B, L, H * d, generator=g).cuda()
    key_mask = torch.ones(B, L)
    if with_mask:
        key_mask[1, 77:] = 0
    key_mask = key_mask.cuda()
    split = lambda x: x.view(B, L, H, d).transpose(1, 2)
    # (a) views in, merged output out
    out_v, _ = mod(*(split(x) for x in proj), key_mask, mat)
    assert out_v.transpose(1, 2).is_contiguous()           # [B, L, H, d] memory: merging the heads is a view
    merged = out_v.transpose(1, 2).reshape(B, L, H * d)
    assert merged.data_ptr() == out_v.data_ptr()
    merged.backward(dmerged)
    grads_v = [x.grad.clone() for x in proj]
    for x in proj:
        x.grad = None
    # (b) contiguous copies in
    out_c, _ = mod(*(split(x).contiguous() for x in proj), key_mask, mat)
    assert out_c.is_contiguous()
    out_c.transpose(1, 2).reshape(B, L, H * d).backward(dmerged)
    assert torch.equal(out_v, out_c)
    for a, x in zip(grads_v, proj):
        assert torch.equal(a, x.grad)
    # and against the float64 model of the layer
    qc, kc, vc = (split(x.detach().double().cpu()).requires_grad_() for x in proj)
    pat = torch.from_numpy(np.repeat(np.repeat(mat_np, bs, 0), bs, 1)).double()
    O, _ = osa.dense_masked_attention(qc, kc, vc, pat, key_mask.double().cpu() if with_mask else None)
    O.backward(split(dmerged.double().cpu()))
    assert_close(out_v.detach().cpu().numpy(), O.detach().numpy(), what="views: out")
    for name, a, b in zip(("dq", "dk", "dv"), grads_v, (qc, kc, vc)):
        assert_close(split(a).cpu().numpy(), b.grad.numpy(), what=f"views: {name}")


# ---------------------------------------------------------------------------------- error handling (host side)
def test_inconsistent_csr_is_reported_not_launched():
    from spion_amd import _lib

    L, d, NB = 64, 32, 1
    abi = SparseABI(d, L, NB, 32, with_mask=False)
    sm, off, col = osa.build_csr_from_block_mask(np.eye(2, dtype=np.float32), 32)
    bad = col.copy()
    bad[5] = 9999
    abi.set_pattern(sm, off, bad)
    Q, K, V, dO = _inputs(NB, L, d, seed=1)
    with pytest.raises(_lib.SpionLibraryError, match="out of range"):
        abi.forward(Q, K, V)
    off2 = off.copy()
    off2[-1] += 1
    abi.set_pattern(sm, off2, col)
    abi.nnz = int(off[-1])
    with pytest.raises(_lib.SpionLibraryError, match="do not match"):
        abi.forward(Q, K, V)
    abi.close()


# ---------------------------------------------------------------------------------- output cache of the tile path
def test_backward_row_sums_with_and_without_output_cache():
    """The backward gets its row sums either from the handle's copy of O (P pointer known) or from an extra
    sweep (unknown P pointer, copies switched off).  Two forwards in flight (siamese use) must not mix."""
    from spion_amd import _lib
    from tests.abi_utils import oracle_fwd_bwd

    L, bs, d, NB = 256, 32, 32, 3
    mat = _random_block_mask(L // bs, 0.35, seed=77)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    QA, KA, VA, dOA = _inputs(NB, L, d, seed=20)
    QB, KB, VB, dOB = _inputs(NB, L, d, seed=21)
    refA = oracle_fwd_bwd(QA, KA, VA, dOA, sm, off, col)
    refB = oracle_fwd_bwd(QB, KB, VB, dOB, sm, off, col)
    OA, PA = abi.forward(QA, KA, VA)
    OB, PB = abi.forward(QB, KB, VB)          # second forward before the first backward
    gA = abi.backward(QA, KA, VA, PA, dOA)    # copy of O filed under PA
    gB = abi.backward(QB, KB, VB, PB, dOB)
    gA2 = abi.backward(QA, KA, VA, PA.clone(), dOA)   # unknown pointer -> two-sweep kernel
    _lib.core().spion_use_output_cache(abi.handle, 0)
    OA3, PA3 = abi.forward(QA, KA, VA)
    gA3 = abi.backward(QA, KA, VA, PA3, dOA)
    gA4 = abi.backward_with_out(QA, KA, VA, PA3, OA3, dOA)   # no copies kept: the caller hands Out over
    for got, ref, tag in ((gA, refA, "A cached"), (gB, refB, "B cached"), (gA2, refA, "A clone"), (gA3, refA, "A off"),
                          (gA4, refA, "A with Out")):
        for name, t in zip(("dQ", "dK", "dV"), got):
            assert_close(t.cpu().numpy(), ref[name], what=f"{tag} {name}")
    abi.close()


@pytest.mark.parametrize("kind,d,with_mask", [("tile", 32, False), ("tile", 32, True), ("tile", 64, False),
                                              ("tile_rows", 32, False), ("element", 32, True), ("element", 128, False)])
def test_rowmajor_entry_points_match_oracle(kind, d, with_mask):
    """spion_attn_forward_rowmajor / spion_attn_backward_rowmajor: K and V as they are, Out handed to the backward
    (and, once, withheld: the backward then finds the row sums itself).  "tile_rows": long rows, the two-sweep
    forward; 2048 rows and more: one wavefront per row."""
    NB = 3
    if kind == "element":
        L = 150
        sm, off, col = _random_element_csr(L, 0.3, seed=d)
        bs = 1
    else:
        L, bs = (2048, 32) if kind == "tile_rows" else (256, 32)
        mat = _random_block_mask(L // bs, 0.3, seed=d + 1)
        if kind == "tile_rows":
            mat[3, :] = 1   # 64 tiles in one row: beyond what four wavefronts keep in registers
            NB = 1
        sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _inputs(NB, L, d, seed=31, scale=1.3)
    pen = None
    if with_mask:
        valid = torch.tensor([L, L - 40, L // 2][:NB])
        pen = (1e6 * (torch.arange(L)[None, :] >= valid[:, None]).float()).contiguous().cuda()
    ref = oracle_fwd_bwd(Q, K, V, dO, sm, off, col, pen)
    O, P = abi.forward_rowmajor(Q, K, V, pen)
    grads = abi.backward_rowmajor(Q, K, V, P, O, dO)
    grads_no_out = abi.backward_rowmajor(Q, K, V, P, None, dO)
    torch.cuda.synchronize()
    assert abi.last_path() == (2 if kind == "element" else 1)
    assert_close(P.cpu().numpy(), ref["P"], what=f"{kind} d={d} P")
    assert_close(O.cpu().numpy(), ref["O"], what=f"{kind} d={d} O")
    for got, tag in ((grads, "with Out"), (grads_no_out, "without Out")):
        for name, t in zip(("dQ", "dK", "dV"), got):
            assert_close(t.cpu().numpy(), ref[name], what=f"{kind} d={d} {tag} {name}")
    abi.close()


def _head_views(B, H, L, d, layout, n, seed, fill=None):
    """n tensors seen as [B, H, L, d], in memory as the layer has them: "proj": each a [B, L, H*d] projection;
    "fused": slices of one [B, L, n, H, d+4] buffer (one GEMM for all, padded rows); "plain": contiguous."""
    g = torch.Generator().manual_seed(seed)
    if layout == "plain":
        bufs = [torch.randn(B, H, L, d, generator=g).cuda() for _ in range(n)]
        views = bufs
    elif layout == "proj":
        bufs = [torch.randn(B, L, H * d, generator=g).cuda() for _ in range(n)]
        views = [b.view(B, L, H, d).transpose(1, 2) for b in bufs]
    else:
        buf = torch.randn(B, L, n, H, d + 4, generator=g).cuda()
        bufs = [buf]
        views = [buf[:, :, i, :, :d].transpose(1, 2) for i in range(n)]
    if fill is not None:
        for b in bufs:
            b.fill_(fill)
    return bufs, views


@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("layout,kind,with_mask", [("proj", "tile", False), ("fused", "tile", True), ("plain", "tile", False),
                                                   ("proj", "tile_rows", False), ("fused", "many_rows", False)])
def test_strided_entry_points(layout, kind, with_mask, d):
    """spion_attn_forward_strided / spion_attn_backward_strided: heads read and written in place in the memory of
    [B, L, H*d] projections.  Same kernels, same arithmetic as the row-major entry points on contiguous copies:
    bit-identical results; padding between the heads' rows is left alone."""
    H, bs = 2, 32
    B, L = {"tile": (2, 256), "tile_rows": (1, 2048), "many_rows": (8 if d == 32 else 4, 4096)}[kind]
    NB = B * H
    mat = _random_block_mask(L // bs, 0.3 if kind != "many_rows" else 0.05, seed=7)
    if kind == "tile_rows":
        mat[3, :] = 1
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    _, (q, k, v) = _head_views(B, H, L, d, layout, 3, seed=41)
    _, (dout,) = _head_views(B, H, L, d, "proj" if layout != "plain" else "plain", 1, seed=42)
    obufs, (out,) = _head_views(B, H, L, d, "proj" if layout != "plain" else "plain", 1, seed=0, fill=float("nan"))
    gbufs, (dq, dk, dv) = _head_views(B, H, L, d, layout, 3, seed=0, fill=-7.0)
    pen = None
    if with_mask:
        valid = torch.tensor([L, L - 40, L // 2, L - 1][:NB])
        pen = (1e6 * (torch.arange(L)[None, :] >= valid[:, None]).float()).contiguous().cuda()
    P = abi.forward_strided(q, k, v, out, pen)
    abi.backward_strided(q, k, v, P, out, dout, dq, dk, dv)
    torch.cuda.synchronize()
    assert abi.last_path() == 1
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    Qc, Kc, Vc, dOc = flat(q), flat(k), flat(v), flat(dout)
    O2, P2 = abi.forward_rowmajor(Qc, Kc, Vc, pen)
    g2 = abi.backward_rowmajor(Qc, Kc, Vc, P2, O2, dOc)
    torch.cuda.synchronize()
    assert torch.equal(P, P2) and torch.equal(flat(out), O2)
    for name, a, b in zip(("dQ", "dK", "dV"), (dq, dk, dv), g2):
        assert torch.equal(flat(a), b), name
    if layout == "fused":
        assert (gbufs[0][..., d:] == -7.0).all(), "padding between the heads' rows was written"
    if kind != "many_rows":
        ref = oracle_fwd_bwd(Qc, Kc, Vc, dOc, sm, off, col, pen)
        assert_close(P.cpu().numpy(), ref["P"], what=f"strided {layout} P")
        assert_close(flat(out).cpu().numpy(), ref["O"], what=f"strided {layout} O")
        for name, a in zip(("dQ", "dK", "dV"), (dq, dk, dv)):
            assert_close(flat(a).cpu().numpy(), ref[name], what=f"strided {layout} {name}")
    abi.close()


@pytest.mark.parametrize("kind,d,layout,with_mask", [("hybrid", 32, "proj", False), ("hybrid", 32, "fused", True),
                                                     ("hybrid4", 32, "proj", False),
                                                     ("element", 16, "proj", False), ("element", 32, "fused", True),
                                                     ("element", 64, "proj", False), ("element", 128, "fused", False)])
def test_strided_entry_points_on_element_sparse_patterns(kind, d, layout, with_mask):
    """The strided entry points on patterns that are not made of 32x32 tiles: the hybrid kernels (window + random
    entries; "hybrid4": strips of more than six dense tiles, four wavefronts per strip) and the element kernels
    (any head size) read the heads in place too.  Bit-identical to the row-major entry points on contiguous
    copies, both against the oracle."""
    B, H = 2, 2
    NB = B * H
    if kind == "hybrid":
        L = 512
        sm, off, col = workloads.window_random_csr(L, 48, 150, seed=9)
    elif kind == "hybrid4":
        L = 512
        sm, off, col = workloads.window_random_csr(L, 150, 330, seed=4)
    else:
        L = 256
        sm, off, col = workloads.window_random_csr(L, 2, 23, seed=5)
    abi = SparseABI(d, L, NB, 1, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    _, (q, k, v) = _head_views(B, H, L, d, layout, 3, seed=51)
    _, (dout,) = _head_views(B, H, L, d, "proj", 1, seed=52)
    _, (out,) = _head_views(B, H, L, d, "proj", 1, seed=0, fill=float("nan"))
    gbufs, (dq, dk, dv) = _head_views(B, H, L, d, layout, 3, seed=0, fill=-7.0)
    pen = None
    if with_mask:
        valid = torch.tensor([L, L - 40, L // 2, L - 1][:NB])
        pen = (1e6 * (torch.arange(L)[None, :] >= valid[:, None]).float()).contiguous().cuda()
    P = abi.forward_strided(q, k, v, out, pen)
    path = abi.last_path()
    abi.backward_strided(q, k, v, P, out, dout, dq, dk, dv)
    torch.cuda.synchronize()
    assert path == abi.last_path() == (2 if kind == "element" else 3)
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    Qc, Kc, Vc, dOc = flat(q), flat(k), flat(v), flat(dout)
    O2, P2 = abi.forward_rowmajor(Qc, Kc, Vc, pen)
    g2 = abi.backward_rowmajor(Qc, Kc, Vc, P2, O2, dOc)
    torch.cuda.synchronize()
    assert torch.equal(P, P2) and torch.equal(flat(out), O2)
    for name, a, b in zip(("dQ", "dK", "dV"), (dq, dk, dv), g2):
        assert torch.equal(flat(a), b), name
    if layout == "fused":
        assert (gbufs[0][..., d:] == -7.0).all(), "padding between the heads' rows was written"
    ref = oracle_fwd_bwd(Qc, Kc, Vc, dOc, sm, off, col, pen)
    assert_close(P.cpu().numpy(), ref["P"], what=f"strided {kind} P")
    assert_close(flat(out).cpu().numpy(), ref["O"], what=f"strided {kind} O")
    for name, a in zip(("dQ", "dK", "dV"), (dq, dk, dv)):
        assert_close(flat(a).cpu().numpy(), ref[name], what=f"strided {kind} {name}")
    abi.close()


@pytest.mark.parametrize("bs,layout", [(64, "plain"), (64, "fused"), (128, "proj")])
def test_entry_points_agree_on_blocks_of_64_and_larger(bs, layout):
    """Masks of 64 x 64 blocks and larger through the three ways into the backward (transposed-operand ABI, row-major,
    strided heads): the same arithmetic in the same order, bit-identical gradients, and against the oracle."""
    B, H, L, d = 2, 2, 1024, 32
    NB = B * H
    mat = _random_block_mask(L // bs, 0.3, seed=11)
    mat[0, :] = 1  # one long pair of strips
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    _, (q, k, v) = _head_views(B, H, L, d, layout, 3, seed=61)
    _, (dout,) = _head_views(B, H, L, d, "proj" if layout != "plain" else "plain", 1, seed=62)
    _, (out,) = _head_views(B, H, L, d, "proj" if layout != "plain" else "plain", 1, seed=0, fill=float("nan"))
    _, (dq, dk, dv) = _head_views(B, H, L, d, layout, 3, seed=0, fill=-7.0)
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    Qc, Kc, Vc, dOc = flat(q), flat(k), flat(v), flat(dout)
    O1, P1 = abi.forward(Qc, Kc, Vc)
    g1 = abi.backward_with_out(Qc, Kc, Vc, P1, O1, dOc)          # transposed V
    g2 = abi.backward_rowmajor(Qc, Kc, Vc, P1, O1, dOc)          # row-major V
    P = abi.forward_strided(q, k, v, out)
    abi.backward_strided(q, k, v, P, out, dout, dq, dk, dv)      # strided heads
    torch.cuda.synchronize()
    assert torch.equal(P, P1) and torch.equal(flat(out), O1)
    for name, a, b, c in zip(("dQ", "dK", "dV"), g1, g2, (dq, dk, dv)):
        assert torch.equal(a, b), name
        assert torch.equal(a, flat(c)), name
    ref = oracle_fwd_bwd(Qc, Kc, Vc, dOc, sm, off, col, None)
    for name, a in zip(("dQ", "dK", "dV"), g2):
        assert_close(a.cpu().numpy(), ref[name], what=f"blocks of {bs} {name}")
    abi.close()


def test_strided_entry_points_refuse_what_they_cannot_serve():
    import ctypes
    from spion_amd import _lib
    L, bs, B, H = 128, 32, 1, 2
    mat = _random_block_mask(L // bs, 0.5, seed=3)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)

    def call(abi, q, out, heads=H, lin=None):
        P = torch.zeros(abi.NB * abi.nnz, device="cuda")
        lin = lin or _lib.head_layout(q)
        lout = _lib.head_layout(out)
        _lib.core().spion_attn_forward_strided(
            abi.handle, q.data_ptr(), q.data_ptr(), q.data_ptr(), None, P.data_ptr(), out.data_ptr(),
            abi.offsets.data_ptr(), abi.columns.data_ptr(), abi.sum_mat.data_ptr(), abi.nnz, heads,
            ctypes.addressof(lin), ctypes.addressof(lout))

    abi = SparseABI(32, L, B * H, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    q = torch.zeros(B, H, L, 32, device="cuda")
    call(abi, q, torch.zeros_like(q), heads=3)
    with pytest.raises(RuntimeError, match="does not divide"):
        _lib.check_error("heads")
    call(abi, q, torch.zeros_like(q), lin=_lib.HeadLayout(H * L * 32, L * 32, 30))
    with pytest.raises(RuntimeError, match="multiples of 4"):
        _lib.check_error("row stride")
    assert _lib.head_layout(torch.zeros(B, H, L, 33, device="cuda")[..., 1:]) is None   # 4-byte offset
    # inputs may share memory between heads (one K/V head for all query heads), outputs may not
    shared = q[:, :1].expand(B, H, L, 32)
    call(abi, shared, torch.zeros_like(q))
    _lib.check_error("shared input heads")
    call(abi, q, shared)
    with pytest.raises(RuntimeError, match="two elements to one address"):
        _lib.check_error("aliased output")
    abi.close()


@pytest.mark.parametrize("shape", [(3, 512, 32), (2, 256, 64), (2, 100, 32), (1, 70, 45), (4, 2, 1024, 32)])
def test_library_transpose_is_exact(shape):
    from spion_amd import _lib
    x = torch.randn(*shape, device="cuda")
    got = _lib.transpose_last2(x)
    assert got.is_contiguous() and torch.equal(got, x.transpose(-1, -2).contiguous())
