"""spion_attn_backward_noalloc (the entry point that allocates nothing) against spion_attn_backward_rowmajor, bit
for bit, through the C ABI: two calls in a row, the second on a smaller problem (GPU box only); argument checks
(no GPU needed)."""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from spion_amd import _lib
from tests.abi_utils import SparseABI, assert_close, oracle_fwd_bwd


def _case(L, bs, NB, p, seed, with_mask, global_strips=False):
    d = 32
    rng = np.random.default_rng(seed)
    nb = L // bs
    mat = (rng.random((nb, nb)) < p).astype(np.float32)
    mat[np.arange(nb), np.arange(nb)] = 1
    if global_strips:
        mat[0, :] = 1
        mat[:, 0] = 1
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = SparseABI(d, L, NB, bs, with_mask=with_mask)
    abi.set_pattern(sm, off, col)
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(NB, L, d, generator=g).cuda() for _ in range(4))
    pen = None
    if with_mask:
        keep = (torch.arange(L)[None, :] < torch.randint(L // 2, L + 1, (NB, 1), generator=g)).float()
        pen = (1e6 * (1.0 - keep)).cuda().contiguous()
    return abi, (sm, off, col), (Q, K, V, dO), pen


def _noalloc_backward(abi, Q, K, V, P, O, dO):
    dQ, dK, dV = (torch.full((abi.NB, abi.L, abi.d), float("nan"), device="cuda") for _ in range(3))
    _lib.core().spion_attn_backward_noalloc(
        abi.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), P.contiguous().data_ptr(), O.data_ptr(), dO.data_ptr(),
        dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(), abi.offsets.data_ptr(), abi.columns.data_ptr(),
        abi.sum_mat.data_ptr(), abi.nnz)
    _lib.check_error("spion_attn_backward_noalloc")
    return dQ, dK, dV


@pytest.mark.gpu
def test_noalloc_backward_matches_rowmajor_backward_twice():
    """First a larger problem, then a smaller one (which leaves the tail of the shared scratch array holding the
    first call's row sums): both bit-identical to the allocating entry point, the second also against the oracle."""
    for L, bs, NB, p, seed, with_mask in ((1024, 32, 16, 0.15, 1, False), (256, 64, 3, 0.5, 2, True)):
        abi, (sm, off, col), (Q, K, V, dO), pen = _case(L, bs, NB, p, seed, with_mask)
        O, P = abi.forward_rowmajor(Q, K, V, pen)
        want = abi.backward_rowmajor(Q, K, V, P, O, dO)
        got = _noalloc_backward(abi, Q, K, V, P, O, dO)
        torch.cuda.synchronize()
        assert abi.last_path() == 1
        for name, g_, w_ in zip(("dQ", "dK", "dV"), got, want):
            assert torch.equal(g_, w_), f"L={L}: {name} of the no-alloc entry differs from spion_attn_backward_rowmajor"
        if L <= 256:
            ref = oracle_fwd_bwd(Q, K, V, dO, sm, off, col, penalty=pen)
            for name, g_ in zip(("dQ", "dK", "dV"), got):
                assert_close(g_.cpu().numpy(), ref[name], what=f"no-alloc {name}")
        abi.close()


@pytest.mark.gpu
def test_noalloc_backward_on_a_pattern_with_global_strips():
    """A block row and a block column that span the sequence: the allocating entry point runs the long strips and the
    others as two launches on two streams, this one as the same two launches one after the other on the caller's
    stream (it creates no stream either).  Same kernels, same split: bit-identical results."""
    abi, _, (Q, K, V, dO), pen = _case(2048, 32, 4, 0.05, 5, False, global_strips=True)
    O, P = abi.forward_rowmajor(Q, K, V, pen)
    want = abi.backward_rowmajor(Q, K, V, P, O, dO)
    got = _noalloc_backward(abi, Q, K, V, P, O, dO)
    torch.cuda.synchronize()
    assert abi.last_path() == 1
    for name, g_, w_ in zip(("dQ", "dK", "dV"), got, want):
        assert torch.equal(g_, w_), f"{name} of the no-alloc entry differs from spion_attn_backward_rowmajor"
    abi.close()


@pytest.mark.gpu
def test_noalloc_backward_allocates_nothing():
    """What the entry point is for: the call analyses no pattern, leaves the device's free memory where it was and
    can be recorded into a HIP graph (a hipMalloc on the capturing thread would invalidate the capture); every
    replay equals the allocating entry point bit for bit."""
    abi, _, (Q, K, V, dO), _ = _case(512, 32, 4, 0.2, 5, False)
    core = _lib.core()
    O, P = abi.forward_rowmajor(Q, K, V)
    want = abi.backward_rowmajor(Q, K, V, P, O, dO)
    P = P.contiguous()
    dQ, dK, dV = (torch.full((abi.NB, abi.L, abi.d), float("nan"), device="cuda") for _ in range(3))

    def call():
        core.spion_attn_backward_noalloc(
            abi.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), P.data_ptr(), O.data_ptr(), dO.data_ptr(),
            dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(), abi.offsets.data_ptr(), abi.columns.data_ptr(),
            abi.sum_mat.data_ptr(), abi.nnz)
        _lib.check_error("spion_attn_backward_noalloc")

    torch.cuda.synchronize()
    counters = [core.spion_debug_counter(abi.handle, w) for w in (0, 1, 2)]
    free_before = torch.cuda.mem_get_info()[0]
    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    assert [core.spion_debug_counter(abi.handle, w) for w in (0, 1, 2)] == counters, "the call analysed or grew something"
    for name, g_, w_ in zip(("dQ", "dK", "dV"), (dQ, dK, dV), want):
        assert torch.equal(g_, w_), name

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        core.spion_set_stream(abi.handle, torch.cuda.current_stream().cuda_stream)
        call()
    core.spion_set_stream(abi.handle, None)
    for rep in range(3):
        for t in (dQ, dK, dV):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, g_, w_ in zip(("dQ", "dK", "dV"), (dQ, dK, dV), want):
            assert torch.equal(g_, w_), f"replay {rep}: {name}"
    abi.close()


@pytest.mark.gpu
def test_noalloc_backward_refuses_unknown_patterns_and_element_patterns():
    abi, (sm, off, col), (Q, K, V, dO), _ = _case(128, 32, 2, 0.5, 3, False)
    P = torch.zeros(abi.NB * abi.nnz, device="cuda")
    O = torch.zeros_like(Q)
    # never analysed on this handle: the entry point must not analyse (that allocates)
    with pytest.raises(_lib.SpionLibraryError, match="not been analysed"):
        _noalloc_backward(abi, Q, K, V, P, O, dO)
    # an element-sparse pattern (first row loses one column) is analysed by a forward, then refused here
    col2 = np.delete(col, 0)
    off2 = off.copy()
    off2[1:] -= 1
    sm2 = sm.copy()
    sm2[0] -= 1
    abi.set_pattern(sm2, off2, col2)
    O, P = abi.forward_rowmajor(Q, K, V)
    assert abi.last_path() in (2, 3)
    with pytest.raises(_lib.SpionLibraryError, match="aligned 32x32 tiles"):
        _noalloc_backward(abi, Q, K, V, P, O, dO)
    abi.close()


def test_noalloc_backward_argument_checks_without_gpu():
    """Size limit, head size and null pointers are refused before anything touches a device."""
    core = _lib.core()
    core.spion_clear_error()
    assert core.spion_noalloc_max_rows() == 1 << 20
    big = core.spion_block_init(32, 32768, 64, 32)        # 2^21 rows
    assert big
    one = 1  # any non-null address: the checks below fail before a pointer is used
    core.spion_attn_backward_noalloc(big, one, one, one, one, one, one, one, one, one, one, one, one, 1024)
    with pytest.raises(_lib.SpionLibraryError, match="exceeds"):
        _lib.check_error()
    core.spion_block_destroy(big)
    d64 = core.spion_block_init(64, 128, 2, 32)
    core.spion_attn_backward_noalloc(d64, one, one, one, one, one, one, one, one, one, one, one, one, 1024)
    with pytest.raises(_lib.SpionLibraryError, match="emb_dim 64"):
        _lib.check_error()
    core.spion_attn_backward_noalloc(d64, one, one, one, one, None, one, one, one, one, one, one, one, 1024)
    with pytest.raises(_lib.SpionLibraryError, match="null pointer"):
        _lib.check_error()
    core.spion_block_destroy(d64)
