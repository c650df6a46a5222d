"""Seeded sweep over random shapes and patterns: every kernel family against the float64 oracle.

The fixed cases of the other test files pin the branches one knows about; this sweep draws the block grid, block
size, density, head count and the special rows (empty, global, key-masked) at random, so that combinations nobody
listed -- odd strip counts, work-group lists that do not divide by four, chunked strips next to empty ones --
are exercised as well.  Every draw is reproducible from its seed, which the assertion messages name."""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from tests.abi_utils import SparseABI, run_and_check
from tests.test_gpu_bf16 import BF16ABI, _bf16_inputs, _run_and_check as bf16_run_and_check

pytestmark = pytest.mark.gpu


def _draw(seed, d_choices):
    rng = np.random.default_rng(seed)
    bs = int(rng.choice([32, 32, 64, 128]))
    nb = int(rng.integers(2, 1 + max(2, 768 // bs)))
    L = nb * bs
    d = int(rng.choice(d_choices))
    NB = int(rng.integers(1, 7))
    p = float(rng.choice([0.05, 0.15, 0.4, 0.9]))
    mat = (rng.random((nb, nb)) < p).astype(np.float32)
    mat[np.arange(nb), np.arange(nb)] = 1
    if rng.random() < 0.4:
        mat[int(rng.integers(nb)), :] = 1   # global row
    if rng.random() < 0.4:
        mat[:, int(rng.integers(nb))] = 1   # global column
    if rng.random() < 0.3:
        mat[int(rng.integers(nb)), :] = 0   # empty row
    if rng.random() < 0.3:
        mat[:, int(rng.integers(nb))] = 0   # empty column
    with_mask = bool(rng.random() < 0.5)
    pen = None
    if with_mask:
        valid = rng.integers(1, L + 1, size=NB)
        pen = torch.from_numpy((1e6 * (np.arange(L)[None, :] >= valid[:, None])).astype(np.float32)).cuda()
    scale = float(rng.choice([0.5, 1.5, 3.0]))
    return dict(bs=bs, nb=nb, L=L, d=d, NB=NB, mat=mat, pen=pen, scale=scale,
                tag=f"seed {seed}: L={L} bs={bs} d={d} NB={NB} p={p} mask={with_mask} scale={scale}")


@pytest.mark.parametrize("seed", range(100, 116))
def test_random_fp32_tile_patterns(seed):
    c = _draw(seed, [32, 32, 64])
    sm, off, col = osa.build_csr_from_block_mask(c["mat"], c["bs"])
    abi = SparseABI(c["d"], c["L"], c["NB"], c["bs"], with_mask=c["pen"] is not None)
    abi.set_pattern(sm, off, col)
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(c["NB"], c["L"], c["d"], generator=g).cuda() * s for s in (c["scale"], c["scale"], 1, 1))
    run_and_check(abi, Q, K, V, dO, c["pen"], tag=c["tag"])
    assert abi.last_path() == 1, c["tag"]
    abi.close()


@pytest.mark.parametrize("seed", range(200, 212))
def test_random_bf16_patterns(seed):
    c = _draw(seed, [32, 64])
    sm, off, col = osa.build_csr_from_block_mask(c["mat"], c["bs"])
    abi = BF16ABI(c["d"], c["L"], c["NB"], c["bs"])
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(c["NB"], c["L"], c["d"], seed=seed, scale=min(c["scale"], 1.5))
    bf16_run_and_check(abi, Q, K, V, dO, c["pen"], tag=c["tag"])
    abi.close()


@pytest.mark.parametrize("seed", range(300, 308))
def test_random_element_patterns(seed):
    rng = np.random.default_rng(seed)
    L = int(rng.integers(33, 200))
    d = int(rng.choice([16, 32, 64, 128]))
    NB = int(rng.integers(1, 4))
    p = float(rng.choice([0.05, 0.3, 0.8]))
    keep = rng.random((L, L)) < p
    keep[np.arange(L), np.arange(L)] = True
    if rng.random() < 0.5:
        keep[int(rng.integers(L)), :] = False  # empty row
    sm = keep.sum(1).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(sm)]).astype(np.int32)
    col = np.nonzero(keep)[1].astype(np.int32)
    with_mask = bool(rng.random() < 0.5)
    pen = None
    if with_mask:
        valid = rng.integers(1, L + 1, size=NB)
        pen = torch.from_numpy((1e6 * (np.arange(L)[None, :] >= valid[:, None])).astype(np.float32)).cuda()
    abi = SparseABI(d, L, NB, 1, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(NB, L, d, generator=g).cuda() for _ in range(4))
    run_and_check(abi, Q, K, V, dO, pen, tag=f"seed {seed}: element L={L} d={d} NB={NB} p={p} mask={with_mask}")
    assert abi.last_path() == 2
    abi.close()


@pytest.mark.parametrize("seed", range(400, 408))
def test_random_dense_shapes(seed):
    from oracle import dense_attention as oda
    from tests.abi_utils import assert_close
    from tests.test_gpu_dense import _run_dense

    rng = np.random.default_rng(seed)
    L = 32 * int(rng.integers(1, 40))
    d = int(rng.choice([32, 32, 64]))
    NB = 2 * int(rng.integers(1, 4))
    with_mask = bool(rng.random() < 0.5)
    g = torch.Generator().manual_seed(seed)
    scale = float(rng.choice([0.5, 1.0, 2.0]))
    Q, K, V, dO = (torch.randn(NB, L, d, generator=g).cuda() * s for s in (scale, scale, 1, 1))
    pen = pen_np = None
    if with_mask:
        km = (np.arange(L)[None, :] < rng.integers(1, L + 1, size=NB // 2)[:, None]).astype(np.float32)
        pen_np = osa.key_penalty_from_mask(km, 2)
        pen = torch.from_numpy(pen_np).cuda()
    got = _run_dense(d, L, NB, Q, K, V, dO, pen)
    f = lambda t: t.cpu().numpy().astype(np.float64)
    O, P = oda.dense_attention_forward(f(Q), f(K), f(V), None if pen_np is None else pen_np.astype(np.float64))
    dQ, dK, dV = oda.dense_attention_backward(f(Q), f(K), f(V), P, f(dO))
    for name, ref in (("P", P), ("O", O), ("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(got[name], ref, what=f"seed {seed}: dense L={L} d={d} NB={NB} mask={with_mask} {name}")
