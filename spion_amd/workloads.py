"""Seeded synthetic workloads of the benchmark configurations (shared by bench.py and the tests).

Nothing here touches the GPU kernels; it only produces masks, CSR patterns and input tensors.
"""
from __future__ import annotations

import numpy as np
import torch


def band_random_block_mask(nb: int, band: int, density: float | None = None, extra_frac: float | None = None,
                           seed: int = 1) -> np.ndarray:
    """[nb, nb] float32 0/1: blocks with |I-J| <= band, plus random off-band blocks.

    ``extra_frac``: each off-band block is kept with this probability; or ``density``: off-band blocks are
    drawn (without replacement) until the total fraction of kept blocks reaches ``density``.
    """
    rng = np.random.default_rng(seed)
    I, J = np.meshgrid(np.arange(nb), np.arange(nb), indexing="ij")
    mat = (np.abs(I - J) <= band).astype(np.float32)
    off = np.flatnonzero(mat.ravel() == 0)
    if extra_frac is not None:
        pick = off[rng.random(off.size) < extra_frac]
    else:
        want = int(round(density * nb * nb)) - int(mat.sum())
        pick = rng.choice(off, size=max(0, min(want, off.size)), replace=False)
    mat.ravel()[pick] = 1.0
    return mat


def config1_mask() -> np.ndarray:
    """L=1024, 32x32 blocks: diagonal band of width 3 plus 5 % of the off-band blocks (about 14 %)."""
    return band_random_block_mask(32, 1, extra_frac=0.05, seed=1)


def north_star_mask(block_size: int = 32) -> np.ndarray:
    """L=4096: diagonal band of width 3 plus random blocks up to 10 % block density."""
    return band_random_block_mask(4096 // block_size, 1, density=0.10, seed=1)


def config5_mask() -> np.ndarray:
    """L=16384, 64x64 blocks: diagonal band, one global block row and column, 1 % random blocks (about 3.7 %)."""
    mat = band_random_block_mask(256, 2, extra_frac=0.01, seed=1)
    mat[0, :] = 1.0
    mat[:, 0] = 1.0
    return mat


def window_random_csr(L: int, window: int, per_row: int, seed: int = 3):
    """Element-sparse pattern: columns [i-window, i+window] plus uniform random columns up to
    ``per_row`` entries in every row (sorted, unique).  Returns (sum_mat, offsets, columns) int32."""
    rng = np.random.default_rng(seed)
    cols = np.empty((L, per_row), dtype=np.int32)
    for i in range(L):
        lo, hi = max(0, i - window), min(L, i + window + 1)
        need = per_row - (hi - lo)
        keep = np.zeros(L, dtype=bool)
        keep[lo:hi] = True
        if need > 0:
            cand = np.concatenate([np.arange(0, lo), np.arange(hi, L)])
            keep[rng.choice(cand, size=need, replace=False)] = True
        row = np.flatnonzero(keep)[:per_row]
        cols[i] = row
    sum_mat = np.full(L, per_row, dtype=np.int32)
    offsets = (np.arange(L + 1, dtype=np.int64) * per_row).astype(np.int32)
    return sum_mat, offsets, cols.ravel()


def qkv(batch: int, heads: int, L: int, d: int, scale: float = 1.0, seed: int = 0, device="cpu",
        dtype=torch.float32):
    """Q, K, V ~ N(0,1)*scale and dO ~ N(0,1), generated on the CPU from fixed seeds."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(batch, heads, L, d, generator=g, dtype=torch.float32) * scale for _ in range(3))
    g2 = torch.Generator().manual_seed(seed + 2)
    do = torch.randn(batch, heads, L, d, generator=g2, dtype=torch.float32)
    return tuple(t.to(device=device, dtype=dtype) for t in (q, k, v, do))


def valid_length_mask(batch: int, L: int, lo: int, hi: int, seed: int = 5) -> torch.Tensor:
    """[batch, L] float 0/1 key mask with per-sample valid lengths uniform in [lo, hi]."""
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (batch,), generator=g)
    return (torch.arange(L)[None, :] < lens[:, None]).to(torch.float32)


def score_maps_config2(n_maps: int = 2, L: int = 1024, d: int = 32, seed: int = 0) -> torch.Tensor:
    """Config 2 input: softmax(QK^T/sqrt(d)) for Q, K ~ N(0,1), plus a +3 sigma boost on a seeded
    diagonal band.  [n_maps, L, L] float32 (CPU)."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(n_maps):
        q = torch.randn(L, d, generator=g)
        k = torch.randn(L, d, generator=g)
        a = torch.softmax(q @ k.t() / float(np.sqrt(d)), dim=-1)
        sigma = a.std()
        width = int(torch.randint(8, 40, (1,), generator=g))
        shift = int(torch.randint(-64, 65, (1,), generator=g))
        i = torch.arange(L)[:, None]
        j = torch.arange(L)[None, :]
        band = ((j - i - shift).abs() <= width) | ((j - i).abs() <= 4)
        out.append(a + 3.0 * sigma * band.to(a.dtype))
    return torch.stack(out, 0).contiguous()


def sparse_flops(nnz: int, d: int, nb: int) -> float:
    """Algorithmic FLOPs of one forward+backward: 12 * n * d * NB (softmax excluded)."""
    return 12.0 * nnz * d * nb


def sparse_bytes(nnz: int, L: int, d: int, nb: int) -> float:
    """Algorithmic HBM bytes of one forward+backward in fp32 with P materialised once:
    4*(11*L*d + 2n)*NB plus the shared index 4*(n + 2L)."""
    return 4.0 * (11.0 * L * d + 2.0 * nnz) * nb + 4.0 * (nnz + 2.0 * L)
