"""The library's per-handle cache of analysed patterns and of kept forward outputs, keyed by device addresses:
eviction, address reuse, registration from host arrays (GPU box only)."""
import ctypes

import numpy as np
import pytest
import torch

import spion_amd
from oracle import sparse_attention as osa
from spion_amd import _lib, workloads
from spion_amd.attention import Attention
from spion_amd.csr import CsrCache, index_from_host
from tests.abi_utils import SparseABI, assert_close, oracle_fwd_bwd

pytestmark = pytest.mark.gpu


def _inputs(NB, L, d, seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(NB, L, d, generator=g).cuda() for _ in range(4))


def _two_masks_equal_nnz(nb, seed):
    """Two different block masks with the same number of blocks in every block row (hence equal nnz and equal
    Offsets): the worst case for a cache keyed by (addresses, nnz)."""
    rng = np.random.default_rng(seed)
    a = np.eye(nb, dtype=np.float32)
    b = np.eye(nb, dtype=np.float32)
    for i in range(nb):
        others = [j for j in range(nb) if j != i]
        pa = rng.choice(others, size=2, replace=False)
        pb = rng.choice([j for j in others if j not in pa], size=2, replace=False)
        a[i, pa] = 1
        b[i, pb] = 1
    assert a.sum() == b.sum() and not np.array_equal(a, b)
    return a, b


def test_module_cache_eviction_with_reused_addresses():
    """A module whose mask cache holds one entry alternates between two masks of equal nnz: every eviction frees
    the index tensors, torch hands the same addresses to the next index, and the results must still follow the mask
    in use (the eviction tells the library to forget the key)."""
    B, H, L, d, bs = 1, 2, 256, 32, 32
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    cpp = Attention._blockcuda_compile_module()
    mod = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    mod.csr_cache = CsrCache(capacity=1, handle=mod.attn_handle)
    ma, mb = _two_masks_equal_nnz(L // bs, seed=4)
    mats = [torch.from_numpy(m).cuda() for m in (ma, mb)]
    q, k, v, do = workloads.qkv(B, H, L, d, seed=3, device="cuda")
    ones = torch.ones(B, L, device="cuda")
    seen = set()
    for rnd in range(3):
        for m_np, m in zip((ma, mb), mats):
            qq, kk, vv = (t.detach().clone().requires_grad_() for t in (q, k, v))
            out, p = mod(qq, kk, vv, ones, m)
            out.backward(do)
            idx = mod.csr_cache.get(m, bs)
            seen.add((idx.offsets.data_ptr(), idx.columns.data_ptr()))
            sm, off, col = osa.build_csr_from_block_mask(m_np, bs)
            f = lambda t: t.detach().reshape(B * H, L, d)
            ref = oracle_fwd_bwd(f(q), f(k), f(v), f(do), sm, off, col)
            assert_close(out.detach().reshape(B * H, L, d).cpu().numpy(), ref["O"], what=f"round {rnd} O")
            assert_close(qq.grad.reshape(B * H, L, d).cpu().numpy(), ref["dQ"], what=f"round {rnd} dQ")
            assert_close(kk.grad.reshape(B * H, L, d).cpu().numpy(), ref["dK"], what=f"round {rnd} dK")
    # informational: on this allocator the two indices do end up at the same addresses
    print("distinct (offsets, columns) address pairs seen:", len(seen))


def test_raw_abi_index_rewritten_in_place_needs_forget():
    L, bs, d, NB = 256, 32, 32, 2
    ma, mb = _two_masks_equal_nnz(L // bs, seed=9)
    Q, K, V, dO = _inputs(NB, L, d, seed=5)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    sma, offa, cola = osa.build_csr_from_block_mask(ma, bs)
    smb, offb, colb = osa.build_csr_from_block_mask(mb, bs)
    abi.set_pattern(sma, offa, cola)
    refa = oracle_fwd_bwd(Q, K, V, dO, sma, offa, cola)
    refb = oracle_fwd_bwd(Q, K, V, dO, smb, offb, colb)
    O, _ = abi.forward(Q, K, V)
    assert_close(O.cpu().numpy(), refa["O"], what="first pattern")
    # same arrays, new contents, equal nnz
    abi.offsets.copy_(torch.from_numpy(offb))
    abi.columns.copy_(torch.from_numpy(colb))
    _lib.core().spion_forget_pattern(abi.handle, abi.offsets.data_ptr(), abi.columns.data_ptr())
    O, P = abi.forward(Q, K, V)
    dQ, dK, dV = abi.backward(Q, K, V, P, dO)
    for name, got in (("O", O), ("P", P), ("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(got.cpu().numpy(), refb[name], what=f"rewritten pattern {name}")
    abi.close()


def test_handle_keeps_several_patterns_and_registration_from_host():
    """Eight patterns alternate on one handle; each is analysed once (spion_register_pattern from the host arrays),
    a second registration under the same key replaces the first."""
    L, bs, d, NB = 128, 32, 32, 2
    core = _lib.core()
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    Q, K, V, dO = _inputs(NB, L, d, seed=6)
    pats = []
    for s in range(8):
        rng = np.random.default_rng(100 + s)
        m = (rng.random((L // bs, L // bs)) < 0.5).astype(np.float32)
        m[np.arange(L // bs), np.arange(L // bs)] = 1
        sm, off, col = osa.build_csr_from_block_mask(m, bs)
        idx = index_from_host(sm, off, col, torch.device("cuda"), abi.handle)
        pats.append((sm, off, col, idx))
    for rnd in range(2):
        for sm, off, col, idx in pats:
            abi.sum_mat, abi.offsets, abi.columns, abi.nnz = idx.sum_mat, idx.offsets, idx.columns, idx.nnz
            O, P = abi.forward(Q, K, V)
            ref = oracle_fwd_bwd(Q, K, V, dO, sm, off, col)
            assert_close(O.cpu().numpy(), ref["O"], what="alternating patterns O")
            assert_close(P.cpu().numpy(), ref["P"], what="alternating patterns P")
    # a malformed host index is refused and nothing is filed under the key
    sm, off, col, idx = pats[0]
    bad = col.copy()
    bad[1] = bad[0]
    rc = core.spion_register_pattern(abi.handle, idx.offsets.data_ptr(), idx.columns.data_ptr(), idx.nnz,
                                     off.ctypes.data, bad.ctypes.data)
    assert rc != 0
    assert b"strictly increasing" in core.spion_handle_error(abi.handle)
    with pytest.raises(_lib.SpionLibraryError, match="strictly increasing"):
        _lib.check_error()
    core.spion_clear_handle_error(abi.handle)
    assert core.spion_handle_error(abi.handle) == b""
    abi.close()


def test_kept_output_copy_is_dropped_by_forwards_that_do_not_refresh_it():
    """A forward through the reference ABI files a copy of Out under its P buffer.  A later forward that fills the
    same P buffer without refreshing the copy (strided heads) must drop it: the reference-ABI backward then
    recomputes its row sums instead of taking them from the stale copy."""
    B, H, L, d, bs = 1, 2, 256, 32, 32
    NB = B * H
    rng = np.random.default_rng(3)
    m = (rng.random((L // bs, L // bs)) < 0.4).astype(np.float32)
    m[np.arange(L // bs), np.arange(L // bs)] = 1
    sm, off, col = osa.build_csr_from_block_mask(m, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    Q1, K1, V1, dO = _inputs(NB, L, d, seed=7)
    Q2, K2, V2, _ = _inputs(NB, L, d, seed=8)
    core = _lib.core()
    P = torch.empty(NB * abi.nnz, device="cuda")
    O = torch.empty(NB, L, d, device="cuda")
    K1t = K1.transpose(1, 2).contiguous()
    abi.lib.attn_forward(abi.handle, Q1.data_ptr(), K1t.data_ptr(), V1.data_ptr(), P.data_ptr(), O.data_ptr(),
                         abi.offsets.data_ptr(), abi.columns.data_ptr(), abi.sum_mat.data_ptr(), abi.nnz)
    # second forward into the same P buffer through the strided entry point (no kept copy)
    q2, k2, v2 = (t.view(B, H, L, d) for t in (Q2, K2, V2))
    out2 = torch.empty(B, H, L, d, device="cuda")
    lay = _lib.head_layout(q2)
    core.spion_attn_forward_strided(abi.handle, q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), None, P.data_ptr(),
                                    out2.data_ptr(), abi.offsets.data_ptr(), abi.columns.data_ptr(),
                                    abi.sum_mat.data_ptr(), abi.nnz, H, ctypes.addressof(lay), ctypes.addressof(lay))
    _lib.check_error("forwards")
    dQ, dK, dV = abi.backward(Q2, K2, V2, P.view(NB, abi.nnz), dO)
    ref = oracle_fwd_bwd(Q2, K2, V2, dO, sm, off, col)
    for name, got in (("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(got.cpu().numpy(), ref[name], what=f"backward after a forward that kept no copy: {name}")
    abi.close()
