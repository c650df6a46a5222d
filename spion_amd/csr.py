"""Block mask -> element-level CSR index on the device, cached per mask.

The reference rebuilds the index on every forward call with an O(L^2) nearest-neighbour upsample and
``nonzero()`` plus two device-to-host synchronisations (models/attention_blockcuda.py:26-43).  Here it
is built once per distinct mask (one host round trip) and reused; a cache entry keeps a reference to the
mask tensor, so neither its address nor its version counter can be recycled while the entry lives.

The library analyses an index once per (Offsets address, Columns address, nnz) and trusts that key.  A cache
that belongs to a handle therefore registers every new index with the library straight from its host arrays
(no copy back, no wait for the stream in the first forward) and tells the library to forget an index when its
entry is evicted -- before torch can hand the freed addresses to another index.

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

    def __post_init__(self):
        # (Offsets, Columns, SumMat, nnz) as the C entry points take them; the tensors never change or move
        self.tail = (self.offsets.data_ptr(), self.columns.data_ptr(), self.sum_mat.data_ptr(), self.nnz)


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


def index_from_host(sum_mat: np.ndarray, offsets: np.ndarray, columns: np.ndarray, device, handle=None,
                    keepalive=None) -> CsrIndex:
    """Device copies of a host-built CSR index; with ``handle`` the pattern is registered with the library from
    the host arrays (spion_register_pattern), so that its first use neither copies the index back nor waits."""
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    columns = np.ascontiguousarray(columns, dtype=np.int32)
    sum_mat = np.ascontiguousarray(sum_mat, dtype=np.int32)
    nnz = int(offsets[-1])
    entry = CsrIndex(
        sum_mat=torch.from_numpy(sum_mat).to(device),
        offsets=torch.from_numpy(offsets).to(device),
        columns=torch.from_numpy(columns).to(device) if columns.size else torch.zeros(1, dtype=torch.int32, device=device),
        nnz=nnz,
        keepalive=keepalive,
    )
    if handle:
        from . import _lib

        rc = _lib.core().spion_register_pattern(handle, entry.offsets.data_ptr(), entry.columns.data_ptr(), nnz,
                                                offsets.ctypes.data, columns.ctypes.data if columns.size else None)
        if rc != 0:
            _lib.check_error("spion_register_pattern")
    return entry


class CsrCache:
    """LRU cache: (mask storage address, version, shape, block size) -> CsrIndex.  ``handle``: the sparse handle
    the indices are used with (None: indices are not registered and evictions are not reported)."""

    def __init__(self, capacity: int = 8, handle=None):
        self.capacity = capacity
        self.handle = handle
        self._entries: "OrderedDict[tuple, CsrIndex]" = OrderedDict()

    def _forget(self, entry: CsrIndex) -> None:
        if self.handle:
            from . import _lib

            _lib.core().spion_forget_pattern(self.handle, entry.offsets.data_ptr(), entry.columns.data_ptr())

    def put(self, mat: torch.Tensor, block_size: int, entry: CsrIndex) -> None:
        """File a prebuilt index (a sidecar built when the masks were loaded) under ``mat``."""
        key = (mat.data_ptr(), mat._version, mat.shape, mat.stride(), block_size, mat.device)
        old = self._entries.pop(key, None)
        if old is not None and old is not entry:
            self._forget(old)
        entry.keepalive = mat
        self._entries[key] = entry
        self._trim()

    def _trim(self) -> None:
        while len(self._entries) > self.capacity:
            _, old = self._entries.popitem(last=False)
            self._forget(old)

    def get(self, mat: torch.Tensor, block_size: int) -> CsrIndex:
        key = (mat.data_ptr(), mat._version, mat.shape, mat.stride(), block_size, mat.device)
        hit = self._entries.get(key)
        if hit is not None:
            self._entries.move_to_end(key)
            return hit
        if mat.dim() != 2 or mat.shape[0] != mat.shape[1]:
            raise ValueError(f"block mask must be square [nb, nb], got {tuple(mat.shape)}")
        sum_mat, offsets, columns = block_mask_to_csr_host(mat.detach().cpu().numpy(), block_size)
        entry = index_from_host(sum_mat, offsets, columns, mat.device, self.handle, keepalive=mat)
        self._entries[key] = entry
        self._trim()
        return entry
