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
    assert abi.last_path() in (2, 3)   # gather kernels, or the hybrid kernels when enough 32x32 tiles are well filled
    abi.close()


@pytest.mark.parametrize("seed", range(500, 512))
def test_random_hybrid_patterns(seed):
    """Element-sparse patterns with dense structure, drawn at random: a band of random width (sometimes shifted off
    the diagonal or doubled), a few full blocks, random scattered entries, empty rows and columns, key masks.  Through
    the reference's ABI (kept copy of Out) and the row-major entries (Out handed over): both against the oracle and
    equal to each other bit for bit."""
    from tests.abi_utils import assert_close, oracle_fwd_bwd
    rng = np.random.default_rng(seed)
    L = 32 * int(rng.integers(4, 25))
    NB = int(rng.integers(1, 5))
    keep = np.zeros((L, L), dtype=bool)
    i = np.arange(L)
    w = int(rng.choice([8, 24, 48, 100]))
    shift = int(rng.choice([0, 0, 37]))
    keep |= np.abs(i[:, None] - i[None, :] - shift) <= w
    if rng.random() < 0.4:
        keep |= np.abs(i[:, None] - i[None, :] + L // 3) <= w // 2      # a second band
    for _ in range(int(rng.integers(0, 4))):                            # full blocks anywhere
        a, b, n = int(rng.integers(0, L - 64)), int(rng.integers(0, L - 64)), int(rng.choice([32, 64]))
        keep[a:a + n, b:b + n] = True
    keep |= rng.random((L, L)) < float(rng.choice([0.0, 0.01, 0.04]))   # scattered entries
    if rng.random() < 0.5:
        keep[int(rng.integers(L)), :] = False
    if rng.random() < 0.5:
        keep[:, int(rng.integers(L))] = False
    if rng.random() < 0.3:
        r0 = 32 * int(rng.integers(L // 32))
        keep[r0:r0 + 32, :] = False                                      # an empty strip
    sm = keep.sum(1).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(sm)]).astype(np.int32)
    col = np.nonzero(keep)[1].astype(np.int32)
    with_mask = bool(rng.random() < 0.5)
    pen = None
    if with_mask:
        valid = rng.integers(1, L + 1, size=NB)
        pen = torch.from_numpy((1e6 * (np.arange(L)[None, :] >= valid[:, None])).astype(np.float32)).cuda()
    tag = f"seed {seed}: hybrid L={L} NB={NB} band={w} shift={shift} nnz={int(off[-1])} mask={with_mask}"
    abi = SparseABI(32, L, NB, 1, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    g = torch.Generator().manual_seed(seed)
    scale = float(rng.choice([0.5, 1.5]))
    Q, K, V, dO = (torch.randn(NB, L, 32, generator=g).cuda() * s for s in (scale, scale, 1, 1))
    got, ref = run_and_check(abi, Q, K, V, dO, pen, tag=tag)
    path = abi.last_path()
    assert path in (2, 3), tag
    O2, P2 = abi.forward_rowmajor(Q, K, V, pen)
    g2 = abi.backward_rowmajor(Q, K, V, P2, O2, dO)
    torch.cuda.synchronize()
    assert abi.last_path() == path, tag
    assert torch.equal(P2, got["P"]) and torch.equal(O2, got["O"]), tag
    for name, a in zip(("dQ", "dK", "dV"), g2):
        assert torch.equal(a, got[name]), f"{tag} {name}"
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


def _random_views(rng, B, H, L, d, n, gen, fill=None):
    """n [B, H, L, d] views in one of the memory layouts a layer produces, drawn at random: contiguous, each a
    [B, L, H*d] projection, slices of one fused buffer, the latter two with padded rows."""
    kind = str(rng.choice(["plain", "proj", "fused"]))
    pad = int(rng.choice([0, 4, 12]))
    if kind == "plain":
        views = [torch.randn(B, H, L, d, generator=gen).cuda() for _ in range(n)]
    elif kind == "proj":
        views = [torch.randn(B, L, H, d + pad, generator=gen).cuda()[..., :d].transpose(1, 2) for _ in range(n)]
    else:
        buf = torch.randn(B, L, n, H, d + pad, generator=gen).cuda()
        views = [buf[:, :, i, :, :d].transpose(1, 2) for i in range(n)]
    if fill is not None:
        for v in views:
            v.fill_(fill)
    return kind, views


@pytest.mark.parametrize("seed", range(500, 510))
def test_random_strided_heads(seed):
    """The strided entry points of the sparse and the dense phase on random shapes, patterns and memory layouts:
    bit for bit what the row-major entry points / the reference's ABI give for contiguous copies, which the other
    sweeps hold against the oracle."""
    from spion_amd import _lib
    from spion_amd.attention import Attention
    from tests.test_gpu_dense import _run_dense
    import ctypes

    c = _draw(seed, [32])
    rng = np.random.default_rng(seed + 7)
    H = int(rng.choice([1, 2, 3]))
    B = max(1, c["NB"] // H)
    NB, L, d = B * H, c["L"], 32
    pen = c["pen"]
    if pen is not None:
        pen = pen[:1].repeat(NB, 1).contiguous()
    gen = torch.Generator().manual_seed(seed)
    kq, (q, k, v) = _random_views(rng, B, H, L, d, 3, gen)
    ko, (out, dout) = _random_views(rng, B, H, L, d, 2, gen)
    kg, (dq, dk, dv) = _random_views(rng, B, H, L, d, 3, gen, fill=float("nan"))
    tag = f"{c['tag']} B={B} H={H} layouts {kq}/{ko}/{kg}"
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    # sparse
    sm, off, col = osa.build_csr_from_block_mask(c["mat"], c["bs"])
    abi = SparseABI(d, L, NB, c["bs"], with_mask=pen is not None)
    abi.set_pattern(sm, off, col)
    P = abi.forward_strided(q, k, v, out, pen)
    abi.backward_strided(q, k, v, P, out, dout, dq, dk, dv)
    O2, P2 = abi.forward_rowmajor(flat(q), flat(k), flat(v), pen)
    g2 = abi.backward_rowmajor(flat(q), flat(k), flat(v), P2, O2, flat(dout))
    torch.cuda.synchronize()
    assert torch.equal(P, P2) and torch.equal(flat(out), O2), tag
    for name, a, b in zip(("dQ", "dK", "dV"), (dq, dk, dv), g2):
        assert torch.equal(flat(a), b), f"{tag}: sparse {name}"
    abi.close()
    # dense phase
    lib = Attention._cuda_mask_compile_module() if pen is not None else Attention._cuda_compile_module()
    h = lib.init(d, L, NB)
    _lib.check_error("init")
    attn = torch.full((NB, L, L), float("nan"), device="cuda")
    lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
    A = ctypes.addressof
    core = _lib.core()
    core.spion_dense_forward_strided(h, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen.data_ptr() if pen is not None else None,
                                     attn.data_ptr(), out.data_ptr(), H, A(lin), A(lout))
    _lib.check_error("dense forward strided")
    core.spion_dense_backward_strided(h, q.data_ptr(), k.data_ptr(), v.data_ptr(), attn.data_ptr(), out.data_ptr(),
                                      dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), H, A(lin), A(lout),
                                      A(lgrad))
    _lib.check_error("dense backward strided")
    torch.cuda.synchronize()
    lib.destroy(h)
    ref = _run_dense(d, L, NB, flat(q), flat(k), flat(v), flat(dout), pen)
    got = dict(O=flat(out), P=attn.transpose(1, 2), dQ=flat(dq), dK=flat(dk), dV=flat(dv))
    for name in ("P", "O", "dQ", "dK", "dV"):
        assert np.array_equal(got[name].cpu().numpy(), ref[name]), f"{tag}: dense {name}"
