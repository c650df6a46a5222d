"""Block mask -> element-level CSR index on the device, cached per mask.

The reference rebuilds the index on every forward call with an O(L^2) nearest-neighbour upsample and
``nonzero()`` plus two device-to-host synchronisations (models/attention_blockcuda.py:26-43).  Here it
is built once per distinct mask (one host round trip) and reused; a cache entry keeps a reference to the
mask tensor, so neither its address nor its version counter can be recycled while the entry lives.

Layout produced (all int32, on the mask's device), as the C ABI expects:
  sum_mat [L]   entries per row  = block_size * (non-zero blocks in the row's block row)
  offsets [L+1] exclusive prefix sum of sum_mat
  columns [n]   sorted column indices row after row (one head's worth; the library reads no more)
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class CsrIndex:
    sum_mat: torch.Tensor
    offsets: torch.Tensor
    columns: torch.Tensor
    nnz: int
    keepalive: object = None


def block_mask_to_csr_host(mat: np.ndarray, block_size: int):
    """numpy arrays (sum_mat, offsets, columns) for a [nb, nb] block mask (non-zero = kept)."""
    nz = np.asarray(mat) != 0
    nb = nz.shape[0]
    bs = int(block_size)
    L = nb * bs
    counts = nz.sum(axis=1).astype(np.int64) * bs
    sum_mat = np.repeat(counts, bs).astype(np.int32)
    offsets = np.zeros(L + 1, dtype=np.int64)
    np.cumsum(sum_mat, out=offsets[1:])
    if offsets[-1] >= 2 ** 31:
        raise ValueError("pattern has more than 2^31-1 entries per head")
    inner = np.arange(bs, dtype=np.int32)
    rows = []
    for I in range(nb):
        cols_I = (np.nonzero(nz[I])[0].astype(np.int32)[:, None] * bs + inner[None, :]).ravel()
        rows.append(np.tile(cols_I, bs))
    columns = np.concatenate(rows) if rows else np.zeros(0, dtype=np.int32)
    return sum_mat, offsets.astype(np.int32), columns.astype(np.int32)


class CsrCache:
    """LRU cache: (mask storage address, version, shape, block size) -> CsrIndex."""

    def __init__(self, capacity: int = 8):
        self.capacity = capacity
        self._entries: "OrderedDict[tuple, CsrIndex]" = OrderedDict()

    def get(self, mat: torch.Tensor, block_size: int) -> CsrIndex:
        key = (mat.data_ptr(), mat._version, tuple(mat.shape), tuple(mat.stride()), int(block_size), str(mat.device))
        hit = self._entries.get(key)
        if hit is not None:
            self._entries.move_to_end(key)
            return hit
        if mat.dim() != 2 or mat.shape[0] != mat.shape[1]:
            raise ValueError(f"block mask must be square [nb, nb], got {tuple(mat.shape)}")
        sum_mat, offsets, columns = block_mask_to_csr_host(mat.detach().cpu().numpy(), block_size)
        dev = mat.device
        entry = CsrIndex(
            sum_mat=torch.from_numpy(sum_mat).to(dev),
            offsets=torch.from_numpy(offsets).to(dev),
            columns=torch.from_numpy(columns).to(dev) if columns.size else torch.zeros(1, dtype=torch.int32, device=dev),
            nnz=int(offsets[-1]),
            keepalive=mat,
        )
        self._entries[key] = entry
        while len(self._entries) > self.capacity:
            self._entries.popitem(last=False)
        return entry
