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


def test_grown_workspaces_retire_the_buffers_they_replace():
    """A workspace that follows the pattern's size is replaced, not freed, when a larger pattern arrives: a HIP graph
    recorded with the smaller pattern still has the old address in its kernel nodes.  Checked through the handle's
    bookkeeping (no stale graph is replayed here): the retired count rises by the number of grown buffers, stays put
    when the smaller pattern comes back, and both patterns keep giving the oracle's results."""
    L, d, B, H = 256, 32, 1, 2
    NB = B * H
    core = _lib.core()
    abi = SparseABI(d, L, NB, 1, with_mask=False)
    small = workloads.window_random_csr(L, 40, 60, seed=3)
    large = workloads.window_random_csr(L, 40, 120, seed=4)
    Q, K, V, dO = _inputs(NB, L, d, seed=21)
    q, k, v, do = (t.view(B, H, L, d) for t in (Q, K, V, dO))

    def step(pattern):
        abi.set_pattern(*pattern)
        out = torch.empty(B, H, L, d, device="cuda")
        P = abi.forward_strided(q, k, v, out)
        assert abi.last_path() == 3
        dq, dk, dv = (torch.empty(B, H, L, d, device="cuda") for _ in range(3))
        abi.backward_strided(q, k, v, P, out, do, dq, dk, dv)   # dS scratch and raw logits belong to the handle
        torch.cuda.synchronize()
        ref = oracle_fwd_bwd(Q, K, V, dO, *pattern)
        for name, got in (("O", out), ("dQ", dq), ("dK", dk), ("dV", dv)):
            assert_close(got.reshape(NB, L, d).cpu().numpy(), ref[name], what=name)
        keep.append((abi.sum_mat, abi.offsets, abi.columns))    # the handle's keys must stay unique addresses

    keep = []
    step(small)
    assert core.spion_debug_counter(abi.handle, 2) == 0
    step(large)
    retired = core.spion_debug_counter(abi.handle, 2)
    assert retired >= 1, "the dS scratch of the smaller pattern must be retired, not freed"
    step(small)
    step(large)
    assert core.spion_debug_counter(abi.handle, 2) == retired
    abi.close()


def test_module_backward_allocates_scratch_by_its_own_pattern():
    """forward(hybrid mask), forward(tile mask), backward(tile), backward(hybrid) on one module: the second backward
    needs the dS scratch although the handle's most recent call ran the tile kernels."""
    B, H, L, d = 1, 2, 256, 32
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=1)
    cpp = Attention._blockcuda_compile_module()
    mod = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, 1))
    sm, off, col = workloads.window_random_csr(L, 40, 100, seed=3)
    hyb = np.zeros((L, L), dtype=np.float32)
    hyb[np.repeat(np.arange(L), sm), col] = 1.0
    blocks = workloads.band_random_block_mask(L // 32, 1, extra_frac=0.1, seed=3)
    tile = np.repeat(np.repeat(blocks, 32, 0), 32, 1).astype(np.float32)
    ones = torch.ones(B, L, device="cuda")
    q, k, v, do = workloads.qkv(B, H, L, d, seed=5, device="cuda")
    outs, leaves = [], []
    for pat in (hyb, tile):
        qq, kk, vv = (t.detach().clone().requires_grad_() for t in (q, k, v))
        out, _ = mod(qq, kk, vv, ones, torch.from_numpy(pat).cuda())
        outs.append(out)
        leaves.append((qq, kk, vv))
    outs[1].backward(do)
    outs[0].backward(do)          # used to fail: "the element path needs the dS scratch buffer"
    torch.cuda.synchronize()
    for pat, (qq, kk, vv) in zip((hyb, tile), leaves):
        rows, cols = np.nonzero(pat)
        sm_ = pat.sum(1).astype(np.int32)
        off_ = np.concatenate([[0], np.cumsum(sm_)]).astype(np.int32)
        ref = oracle_fwd_bwd(q.reshape(B * H, L, d), k.reshape(B * H, L, d), v.reshape(B * H, L, d),
                             do.reshape(B * H, L, d), sm_, off_, cols.astype(np.int32))
        for name, t in (("dQ", qq), ("dK", kk), ("dV", vv)):
            assert_close(t.grad.reshape(B * H, L, d).cpu().numpy(), ref[name], what=name)
