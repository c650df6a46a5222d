"""CPU oracle: SPION pattern discovery (conv filter -> block pool -> quantile -> path walk).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

The reference runs this stage on the CPU with PyTorch ops
(main_conv_ff.py:249-299).  ``route="torch"`` below calls the very same
PyTorch CPU routines (``F.conv2d``, ``F.avg_pool2d``, ``torch.quantile``;
PyTorch is a third-party library, not reference code) and so reproduces the
reference's float32 route up to the summation order of the PyTorch build;
``route="fp64"`` evaluates the closed forms in float64 and rounds once.
``decision_margin`` reports how far every comparison the walk performs is
from flipping, which tells whether the two routes must agree.
"""
from __future__ import annotations

import numpy as np


# --------------------------------------------------------------------------
# conv filter + pooling
# --------------------------------------------------------------------------
def conv_diag_closed_form(A: np.ndarray, ksize: int = 31) -> np.ndarray:
    """C[i, j] = sum_{t=-(k//2)}^{k//2} A[i+t, j+t], zero outside the map (float64).

    Closed form of main_conv_ff.py:258-263: cross-correlation with the
    ksize x ksize identity, stride 1, ``padding='same'``.
    Pinned by: brute-force triple loop on small maps and F.conv2d (tests).
    """
    A = np.asarray(A, dtype=np.float64)
    L0, L1 = A.shape
    h = ksize // 2
    C = np.zeros_like(A)
    for t in range(-h, h + 1):
        if t >= 0:
            C[: L0 - t, : L1 - t] += A[t:, t:]
        else:
            C[-t:, -t:] += A[: L0 + t, : L1 + t]
    return C


def block_pool_closed_form(C: np.ndarray, block_size: int) -> np.ndarray:
    """out[I, J] = mean of the bs x bs block (float64). main_conv_ff.py:264-265."""
    C = np.asarray(C, dtype=np.float64)
    bs = int(block_size)
    nb0, nb1 = C.shape[0] // bs, C.shape[1] // bs
    return C[: nb0 * bs, : nb1 * bs].reshape(nb0, bs, nb1, bs).sum(axis=(1, 3)) / float(bs * bs)


def pooled_map(A: np.ndarray, block_size: int, ksize: int = 31, route: str = "fp64") -> np.ndarray:
    """Pooled, filtered score map [nb, nb] as float32.

    ``ksize == 0`` skips the filter (the pool-only generator, main_ff.py:255-257).
    route "torch": literal main_conv_ff.py:258-265 with the installed PyTorch.
    route "fp64" : closed forms in float64, one rounding to float32.
    """
    if route == "torch":
        import torch
        import torch.nn.functional as F

        data = torch.as_tensor(np.asarray(A, dtype=np.float32))
        x = data.unsqueeze(0)
        if ksize:
            kernel = torch.eye(ksize, dtype=torch.float32)[None, None]
            x = F.conv2d(x, kernel, stride=1, padding="same")
        out = F.avg_pool2d(x, (block_size, block_size))[0]
        return out.numpy().copy()
    C = conv_diag_closed_form(A, ksize) if ksize else np.asarray(A, dtype=np.float64)
    return block_pool_closed_form(C, block_size).astype(np.float32)


# --------------------------------------------------------------------------
# threshold
# --------------------------------------------------------------------------
def quantile_linear(values: np.ndarray, q: float):
    """torch.quantile(values, q) for float32 input, restated step by step.

    main_conv_ff.py:268.  PyTorch (aten/src/ATen/native/Sorting.cpp,
    quantile_compute) sorts the flattened values, forms the rank
    ``r = float32(q) * (N-1)`` in float32, takes ``lo = floor(r)``,
    ``hi = ceil(r)``, ``w = r - lo`` and returns ``lerp(sorted[lo], sorted[hi], w)``
    with lerp(a, b, w) = a + w*(b-a) if w < 0.5 else b - (b-a)*(1-w).
    Returns (thresh float32, lo, hi, w).
    Pinned by: torch.quantile and numpy.quantile(method="linear") (tests).
    """
    s = np.sort(np.asarray(values, dtype=np.float32).ravel())
    N = s.size
    r = np.float32(q) * np.float32(N - 1)
    lo = int(np.floor(r))
    hi = int(np.ceil(r))
    w = np.float32(r - np.float32(lo))
    a, b = s[lo], s[hi]
    diff = np.float32(b - a)
    if w < np.float32(0.5):
        t = np.float32(a + np.float32(w * diff))
    else:
        t = np.float32(b - np.float32(diff * np.float32(np.float32(1.0) - w)))
    return t, lo, hi, w


# --------------------------------------------------------------------------
# greedy path walk ("flood fill")
# --------------------------------------------------------------------------
def flood_fill_walk(data: np.ndarray, x: int, y: int, ff_mat: np.ndarray, thresh, trace=None):
    """Iterative restatement of the recursive ``flood_fill`` (main_conv_ff.py:35-62).

    ``data`` is the pooled map with one zero sentinel row and column appended
    ([nb+1, nb+1]); ``ff_mat`` is [nb, nb] and receives data values at marked
    cells.  From (x, y), with D = data[x+1][y], R = data[x][y+1],
    G = data[x+1][y+1]: go down if D > R and D > G, right if not D > R and
    R > G, else diagonally (all comparisons strict, ties fall to the
    diagonal); the cell moved to is marked when its value exceeds ``thresh``;
    stop when x+1 or y+1 reaches the size of ``data``.  The start cell is not
    marked.  A mark outside ``ff_mat`` raises IndexError exactly as the
    reference's tensor indexing would.
    ``trace`` (optional list) collects (a, b) pairs of every comparison made.
    Pinned by: hand-worked grids and a recursive transcription-free check of
    the move rule in tests (tests/test_oracle_pattern.py).
    """
    n0, n1 = data.shape
    while not (x + 1 == n0 or y + 1 == n1):
        D, R, G = data[x + 1][y], data[x][y + 1], data[x + 1][y + 1]
        if trace is not None:
            trace.append((D, R))
        if D > R:
            if trace is not None:
                trace.append((D, G))
            nx, ny = (x + 1, y) if D > G else (x + 1, y + 1)
        else:
            if trace is not None:
                trace.append((R, G))
            nx, ny = (x, y + 1) if R > G else (x + 1, y + 1)
        val = data[nx][ny]
        if trace is not None:
            trace.append((val, thresh))
        if val > thresh:
            if nx >= ff_mat.shape[0] or ny >= ff_mat.shape[1]:
                raise IndexError("flood_fill mark outside the block grid")
            ff_mat[nx][ny] = val
        x, y = nx, ny
    return ff_mat


def mask_from_pooled(pooled: np.ndarray, thresh, trace=None) -> np.ndarray:
    """Seeds, walk, binarise, force the diagonal. main_conv_ff.py:266-278.

    tmp = pooled with a zero last row/column; seeds (0, k) for k = 0..nb-1 then
    (k, 0); mat = (ff_mat > 0); mat[i, i] = 1.  Returns int8 [nb, nb].
    """
    pooled = np.asarray(pooled, dtype=np.float32)
    nb = pooled.shape[0]
    tmp = np.zeros((nb + 1, nb + 1), dtype=np.float32)
    tmp[:-1, :-1] = pooled
    ff = np.zeros((nb, nb), dtype=np.float32)
    for k in range(nb):
        flood_fill_walk(tmp, 0, k, ff, thresh, trace)
    for k in range(nb):
        flood_fill_walk(tmp, k, 0, ff, thresh, trace)
    mat = (ff > 0).astype(np.int8)
    mat[np.arange(nb), np.arange(nb)] = 1
    return mat


def generate_mask_conv_ff(A, block_size: int, threshold: float, ksize: int = 31, route: str = "fp64"):
    """SPION-CF generator (main_conv_ff.py:254-278); ksize=0 gives SPION-F (main_ff.py:253-272).

    Returns (mask int8 [nb, nb], pooled float32 [nb, nb], thresh float32).
    """
    pooled = pooled_map(A, block_size, ksize, route)
    if route == "torch":
        import torch

        thresh = np.float32(torch.quantile(torch.as_tensor(pooled), threshold).item())
    else:
        thresh = quantile_linear(pooled, threshold)[0]
    return mask_from_pooled(pooled, thresh), pooled, thresh


def generate_mask_conv(A, block_size: int, density: float, ksize: int = 31, route: str = "fp64"):
    """SPION-C generator (main_conv.py:236-256): top-k blocks of the pooled map, k =
    int(nb*nb*density - nb), plus the diagonal.  Ties at the k-th value are
    resolved towards the lower flat index here; torch.topk leaves them
    unspecified, so fixtures must not tie there.
    Returns (mask int8, pooled float32, k).
    """
    pooled = pooled_map(A, block_size, ksize, route)
    nb = pooled.shape[0]
    k = int(nb * nb * density - nb)
    flat = pooled.ravel()
    order = np.argsort(-flat, kind="stable")
    mat = np.zeros(nb * nb, dtype=np.int8)
    if k > 0:
        mat[order[:k]] = 1
    mat = mat.reshape(nb, nb)
    mat[np.arange(nb), np.arange(nb)] = 1
    return mat, pooled, k


# --------------------------------------------------------------------------
# how close to a flip is every decision
# --------------------------------------------------------------------------
def decision_margin(pooled: np.ndarray, threshold: float) -> float:
    """Smallest relative gap |a-b| / max(|a|,|b|) over every comparison the walks make
    (D>R, .>G, .>thresh).  Comparisons of two exact zeros (sentinels) are route
    independent and skipped.  The threshold itself moves continuously with the
    pooled values, so its own sensitivity is covered by the .>thresh gaps.  If the margin exceeds the relative error
    of a route's pooled values by a safe factor, every route yields the same
    mask.
    """
    pooled = np.asarray(pooled, dtype=np.float32)
    thresh, lo, hi, _ = quantile_linear(pooled, threshold)
    trace: list = []
    mask_from_pooled(pooled, thresh, trace)
    best = np.inf
    for a, b in trace:
        a = float(a)
        b = float(b)
        if a == 0.0 and b == 0.0:
            continue
        best = min(best, abs(a - b) / max(abs(a), abs(b)))
    return float(best)
