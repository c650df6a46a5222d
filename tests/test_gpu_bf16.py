"""Parity of the bf16 sparse-attention kernels with the float64 oracle, through the C ABI (GPU box only).

The oracle runs on the bf16-rounded inputs in float64.  Tolerance for the bf16 outputs and gradients, 1e-2
relative, read for tensors whose every element carries the 2^-9 rounding of the bf16 result itself (measured
relative L2 error of a correct kernel: 2.3e-3) and whose gradients cancel (dS = P (dP - g)):
  * relative error in the L2 norm <= 1e-2, and
  * no element further from the oracle than 1e-2 * (|ref| + max|ref|).
The fp32 row statistic the forward hands to the backward must agree within 1e-3 absolute (measured 1e-6).
"""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from spion_amd import BlockAttentionBF16, _lib, workloads
from tests.abi_utils import SparseABI

pytestmark = pytest.mark.gpu

REL_TOL_BF16 = 1e-2
LOG2E = 1.4426950408889634


ROW_TOL_BF16 = 2.5e-2


def assert_close_bf16(got, ref, what="", extra=None):
    """Relative L2 error of the tensor within 1e-2, and every element within
        1e-2 |ref|  +  2.5e-2 rms(ref over the element's own row of d values)  +  1e-2 rms(ref over the tensor).
    Measured against the oracle on the cases of this file: the tensor's L2 error is 0.22 - 0.26 % (bf16 rounds the
    result to 2^-9 of the element and P and dS to as much ahead of the second product of each chain), a row's L2
    error at most 1.2 % of the row, and the largest element error beyond 1e-2 |ref| is 2.1 % of its row's RMS.  Rows
    differ in scale by more than ten (a global key column collects a term from every query), which is why the
    tensor's RMS alone does not bound an element's noise (seen: 4 % of it) and its maximum is no bound at all.
    The last term covers rows that are all but zero.  ``extra`` (same shape) is added to the bound: dQ and dK carry
    the term that the rounding of O brings in, see ``_oracle``."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - ref)
    rel_l2 = float(np.sqrt((err * err).sum() / max((ref * ref).sum(), 1e-300)))
    assert rel_l2 <= REL_TOL_BF16, f"{what}: relative L2 error {rel_l2:.3e}"
    row_rms = np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True))
    tol = REL_TOL_BF16 * np.abs(ref) + ROW_TOL_BF16 * row_rms + REL_TOL_BF16 * np.sqrt(np.mean(ref * ref))
    if extra is not None:
        tol = tol + extra
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())}/{bad.size} outside tolerance; worst at {idx}: "
                             f"got {got[idx]!r}, ref {ref[idx]!r}")
    return rel_l2


class BF16ABI:
    def __init__(self, d, L, NB, block_size):
        self.lib = _lib.core()
        self.d, self.L, self.NB = d, L, NB
        self.handle = self.lib.spion_block_bf16_init(d, L, NB, block_size)
        _lib.check_error("spion_block_bf16_init")
        assert self.handle

    def close(self):
        self.lib.spion_block_bf16_destroy(self.handle)
        self.handle = None

    def set_pattern(self, sum_mat, offsets, columns):
        dev = "cuda"
        self.np_pattern = (np.asarray(sum_mat), np.asarray(offsets), np.asarray(columns))
        self.sum_mat = torch.from_numpy(np.ascontiguousarray(sum_mat)).to(dev)
        self.offsets = torch.from_numpy(np.ascontiguousarray(offsets)).to(dev)
        cols = np.ascontiguousarray(columns) if len(columns) else np.zeros(1, np.int32)
        self.columns = torch.from_numpy(cols).to(dev)
        self.nnz = int(offsets[-1])

    def forward(self, Q, K, V, pen=None):
        O = torch.full((self.NB, self.L, self.d), float("nan"), dtype=torch.bfloat16, device="cuda")
        lse = torch.full((self.NB, self.L), float("nan"), dtype=torch.float32, device="cuda")
        self.lib.spion_block_bf16_attn_forward(self.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(),
                                               pen.data_ptr() if pen is not None else None, O.data_ptr(),
                                               lse.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(),
                                               self.sum_mat.data_ptr(), self.nnz)
        _lib.check_error("bf16 forward")
        return O, lse

    def backward(self, Q, K, V, O, lse, dO, pen=None):
        dQ, dK, dV = (torch.full((self.NB, self.L, self.d), float("nan"), dtype=torch.bfloat16, device="cuda")
                      for _ in range(3))
        self.lib.spion_block_bf16_attn_backward(self.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(),
                                                pen.data_ptr() if pen is not None else None, O.data_ptr(),
                                                lse.data_ptr(), dO.data_ptr(), dQ.data_ptr(), dK.data_ptr(),
                                                dV.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(),
                                                self.sum_mat.data_ptr(), self.nnz)
        _lib.check_error("bf16 backward")
        return dQ, dK, dV


def _bf16_inputs(NB, L, d, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return tuple((torch.randn(NB, L, d, generator=g) * s).to(torch.bfloat16).cuda() for s in (scale, scale, 1.0, 1.0))


def _oracle(Q, K, V, dO, sum_mat, offsets, columns, pen=None):
    f = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    q, k, v, do = f(Q), f(K), f(V), f(dO)
    penn = None if pen is None else pen.detach().cpu().numpy().astype(np.float64)
    O, P = osa.csr_attention_forward(q, k, v, offsets, columns, sum_mat, penn)
    dQ, dK, dV, _ = osa.csr_attention_backward(q, k, v, P, do, offsets, columns)
    # row statistic: log2 of the softmax denominator with the row maximum folded in
    NB, L, d = q.shape
    rows = osa.csr_row_index(offsets)
    cols = np.asarray(columns[: int(offsets[-1])], dtype=np.int64)
    lse = np.zeros((NB, L))
    for b in range(NB):
        val = np.einsum("nd,nd->n", q[b][rows], k[b][cols]) * float(np.float32(1) / np.sqrt(np.float32(d)))
        if penn is not None:
            val = val - penn[b][cols]
        big = np.full(L, 0.0 if penn is not None else -100.0)
        np.maximum.at(big, rows, val)
        z = np.zeros(L)
        np.add.at(z, rows, np.exp(val - big[rows]))
        z += (L - np.asarray(sum_mat)) * np.exp(-big)
        lse[b] = (big + np.log(z)) * LOG2E
    # The backward takes g_i = sum_t dO_it O_it from the stored output, which bf16 has rounded by up to 2^-8 of
    # each element: |delta g_i| <= 2^-8 A_i with A_i = sum_t |dO_it O_it|.  Every dS_ij = P_ij (dP_ij - g_i) of the
    # row moves by -P_ij delta g_i together, so to first order
    #     |delta dQ_if| <= scale 2^-8 A_i |sum_j P_ij K_jf|,    |delta dK_jf| <= scale 2^-8 sum_i P_ij A_i |Q_if|.
    # On rows whose softmax is saturated (dP_ij close to g_i) these terms exceed dQ and dK themselves.
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    A = np.abs(do * O).sum(-1) * 2.0 ** -8
    extra_dq = scale * A[:, :, None] * np.abs(osa.csr_spmm(P, k, offsets, columns))
    extra_dk = scale * osa.csr_spmm_t(P * A[:, rows], np.abs(q), offsets, columns)
    return dict(O=O, dQ=dQ, dK=dK, dV=dV, lse=lse, extra=dict(dQ=extra_dq, dK=extra_dk))


def _run_and_check(abi, Q, K, V, dO, pen=None, tag=""):
    sm, off, col = abi.np_pattern
    ref = _oracle(Q, K, V, dO, sm, off, col, pen)
    O, lse = abi.forward(Q, K, V, pen)
    dQ, dK, dV = abi.backward(Q, K, V, O, lse, dO, pen)
    torch.cuda.synchronize()
    got_lse = lse.cpu().numpy().astype(np.float64)
    assert np.isfinite(got_lse).all(), f"{tag}: lse not finite"
    assert np.max(np.abs(got_lse - ref["lse"])) < 1e-3, f"{tag}: lse off by {np.max(np.abs(got_lse - ref['lse']))}"
    for name, t in (("O", O), ("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close_bf16(t.float().cpu().numpy(), ref[name], f"{tag} {name}", extra=ref["extra"].get(name))


def _mask(nb, p, seed, global_block=False, empty_row=None, empty_col=None):
    rng = np.random.default_rng(seed)
    mat = (rng.random((nb, nb)) < p).astype(np.float32)
    mat[np.arange(nb), np.arange(nb)] = 1
    if global_block:
        mat[0, :] = 1
        mat[:, 0] = 1
    if empty_row is not None:
        mat[empty_row, :] = 0
    if empty_col is not None:
        mat[:, empty_col] = 0
    return mat


@pytest.mark.parametrize(
    "L,bs,d,NB,p,glob",
    [
        (128, 32, 32, 3, 0.30, False),
        (256, 32, 64, 2, 0.40, False),
        (256, 64, 64, 2, 0.40, False),   # 64x64 blocks = 2x2 tiles
        (512, 128, 32, 1, 0.50, False),
        (2048, 32, 32, 1, 0.04, True),   # a global row and column: strips walked by four wavefronts together
        (2048, 64, 64, 1, 0.06, True),
    ],
)
def test_bf16_matches_oracle(L, bs, d, NB, p, glob):
    mat = _mask(L // bs, p, seed=L + bs + d, global_block=glob)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=1, scale=1.2)
    _run_and_check(abi, Q, K, V, dO, tag=f"bf16 L={L} bs={bs} d={d}")
    abi.close()


def test_bf16_empty_block_row_and_column_and_large_logits():
    L, bs, d, NB = 256, 32, 32, 2
    mat = _mask(L // bs, 0.4, seed=5, empty_row=2, empty_col=5)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=2, scale=4.0)  # logits of +-50 and more: exercises the running maximum
    _run_and_check(abi, Q, K, V, dO, tag="bf16 empty strips, large logits")
    abi.close()


@pytest.mark.parametrize("d", [32, 64])
def test_bf16_with_key_mask(d):
    L, bs, NB = 256, 32, 4
    mat = _mask(L // bs, 0.5, seed=7)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=3)
    valid = torch.tensor([256, 200, 131, 64])
    key_mask = (torch.arange(L)[None, :] < valid[:, None]).float()
    pen = (1e6 * (1.0 - key_mask)).contiguous().cuda()
    _run_and_check(abi, Q, K, V, dO, pen, tag=f"bf16 key mask d={d}")
    O, _ = abi.forward(Q, K, V, pen)
    assert torch.isfinite(O.float()).all()
    abi.close()


@pytest.mark.parametrize("d", [32, 64])
def test_bf16_long_strips_with_key_mask_and_large_logits(d):
    """A global block row and column are cut into chunks whose partial results a merge kernel combines: the
    chunks of a row see different maxima (logits of +-40) and some lie wholly behind the key mask."""
    L, bs, NB = 2048, 32, 2
    mat = _mask(L // bs, 0.04, seed=11, global_block=True)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=4, scale=3.0)
    valid = torch.tensor([2048, 1000])
    key_mask = (torch.arange(L)[None, :] < valid[:, None]).float()
    pen = (1e6 * (1.0 - key_mask)).contiguous().cuda()
    _run_and_check(abi, Q, K, V, dO, pen, tag=f"bf16 long strips, key mask d={d}")
    abi.close()


@pytest.mark.parametrize("lanes", [3, 8])
@pytest.mark.parametrize("d,bs,with_mask", [(32, 32, True), (64, 64, False), (64, 32, True)])
def test_bf16_few_lanes_walk_many_items_each(monkeypatch, lanes, d, bs, with_mask):
    """With a handful of persistent wavefronts each one walks many strips, chunks and pairs of several heads in a
    row, so every kind of hand-over inside a wavefront's load stream (item to item, head to head, a staged result
    followed by the next item's loads, chunk slots of a long strip) is checked against the oracle.  The lane count
    is read when the pattern is indexed."""
    L, NB = 1024, 5
    mat = _mask(L // bs, 0.10, seed=23 + d + bs, global_block=True, empty_row=3)
    mat[3, 3] = 0
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    monkeypatch.setenv("SPION_BF16_LANES", str(lanes))
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    monkeypatch.delenv("SPION_BF16_LANES")
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=6, scale=1.5)
    pen = None
    if with_mask:
        valid = torch.tensor([1024, 700, 1024, 333, 64])
        pen = (1e6 * (1.0 - (torch.arange(L)[None, :] < valid[:, None]).float())).contiguous().cuda()
    _run_and_check(abi, Q, K, V, dO, pen, tag=f"bf16 {lanes} lanes d={d} bs={bs}")
    abi.close()


def _bf16_head_views(B, H, L, d, layout, n, seed, fill=None):
    """n bf16 tensors seen as [B, H, L, d]: "proj": each a [B, L, H*d] projection; "fused": slices of one
    [B, L, n, H, d+8] buffer (padded rows)."""
    g = torch.Generator().manual_seed(seed)
    if layout == "proj":
        bufs = [torch.randn(B, L, H * d, generator=g).to(torch.bfloat16).cuda() for _ in range(n)]
        views = [b.view(B, L, H, d).transpose(1, 2) for b in bufs]
    else:
        buf = torch.randn(B, L, n, H, d + 8, generator=g).to(torch.bfloat16).cuda()
        bufs = [buf]
        views = [buf[:, :, i, :, :d].transpose(1, 2) for i in range(n)]
    if fill is not None:
        for b in bufs:
            b.fill_(fill)
    return bufs, views


@pytest.mark.parametrize("d,layout,glob,with_mask,bs", [(32, "proj", False, False, 32), (64, "fused", False, True, 32),
                                                        (64, "proj", True, False, 32), (32, "fused", True, True, 32),
                                                        (64, "proj", True, False, 64), (32, "fused", False, True, 64),
                                                        (32, "proj", True, False, 128)])
def test_bf16_strided_entry_points(d, layout, glob, with_mask, bs):
    """spion_block_bf16_attn_{forward,backward}_strided: bf16 heads read and written in place in the memory of
    [B, L, H*d] projections (or of one fused, padded buffer).  Same kernels and arithmetic as the contiguous entry
    points on contiguous copies -- long strips cut into chunks and merged included: bit-identical results; the
    padding between the heads' rows is left alone.  With blocks of 64 x 64 and larger the contiguous forward takes two
    strips per wavefront and the strided one a strip per wavefront: two kernels, the same arithmetic in the same
    order."""
    import ctypes
    B, H, L = 2, 2, 1024
    NB = B * H
    mat = _mask(L // bs, 0.1, seed=21, global_block=glob)
    sm, off, col = osa.build_csr_from_block_mask(mat, bs)
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    _, (q, k, v) = _bf16_head_views(B, H, L, d, layout, 3, seed=71)
    _, (dout,) = _bf16_head_views(B, H, L, d, "proj", 1, seed=72)
    _, (out,) = _bf16_head_views(B, H, L, d, "proj", 1, seed=0, fill=float("nan"))
    gbufs, (dq, dk, dv) = _bf16_head_views(B, H, L, d, layout, 3, seed=0, fill=-7.0)
    pen = None
    if with_mask:
        valid = torch.tensor([L, L - 40, L // 2, L - 1])
        pen = (1e6 * (torch.arange(L)[None, :] >= valid[:, None]).float()).contiguous().cuda()
    pen_ptr = pen.data_ptr() if pen is not None else None
    lse = torch.full((NB, L), float("nan"), device="cuda")
    lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
    assert lin is not None and lout is not None and lgrad is not None
    tail = (abi.offsets.data_ptr(), abi.columns.data_ptr(), abi.sum_mat.data_ptr(), abi.nnz)
    abi.lib.spion_block_bf16_attn_forward_strided(abi.handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                                  out.data_ptr(), lse.data_ptr(), *tail, H, ctypes.addressof(lin),
                                                  ctypes.addressof(lout))
    _lib.check_error("bf16 forward strided")
    abi.lib.spion_block_bf16_attn_backward_strided(abi.handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                                   out.data_ptr(), lse.data_ptr(), dout.data_ptr(), dq.data_ptr(),
                                                   dk.data_ptr(), dv.data_ptr(), *tail, H, ctypes.addressof(lin),
                                                   ctypes.addressof(lout), ctypes.addressof(lgrad))
    _lib.check_error("bf16 backward strided")
    torch.cuda.synchronize()
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    Qc, Kc, Vc, dOc = flat(q), flat(k), flat(v), flat(dout)
    O2, lse2 = abi.forward(Qc, Kc, Vc, pen)
    g2 = abi.backward(Qc, Kc, Vc, O2, lse2, dOc, pen)
    torch.cuda.synchronize()
    assert torch.equal(flat(out), O2) and torch.equal(lse, lse2)
    for name, a, b in zip(("dQ", "dK", "dV"), (dq, dk, dv), g2):
        assert torch.equal(flat(a), b), name
    if layout == "fused":
        assert (gbufs[0][..., d:] == -7.0).all(), "padding between the heads' rows was written"
    ref = _oracle(Qc, Kc, Vc, dOc, sm, off, col, pen)
    for name, t in (("O", out), ("dQ", dq), ("dK", dk), ("dV", dv)):
        assert_close_bf16(flat(t).float().cpu().numpy(), ref[name], f"bf16 strided {name}", extra=ref["extra"].get(name))
    # a layout the kernels cannot take is refused
    bad = _lib.HeadLayout(lin.batch_stride, lin.head_stride, lin.row_stride + 4)
    abi.lib.spion_block_bf16_attn_forward_strided(abi.handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen_ptr,
                                                  out.data_ptr(), lse.data_ptr(), *tail, H, ctypes.addressof(bad),
                                                  ctypes.addressof(lout))
    with pytest.raises(RuntimeError, match="multiples of 8"):
        _lib.check_error("bad layout")
    abi.close()


def test_bf16_module_reads_views_in_place():
    """BlockAttentionBF16 on heads that are views of bf16 projections: same values and gradients as on contiguous
    copies (bit-identical: same kernels), output and gradients laid out like the inputs."""
    from spion_amd import BlockAttentionBF16
    B, H, L, d, bs = 2, 2, 512, 64, 64
    mat = torch.from_numpy(_mask(L // bs, 0.3, seed=5).astype(np.float32)).cuda()
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    mod = BlockAttentionBF16(cfg)
    g = torch.Generator().manual_seed(9)
    proj = [torch.randn(B, L, H * d, generator=g).to(torch.bfloat16).cuda().requires_grad_() for _ in range(3)]
    views = [p.view(B, L, H, d).transpose(1, 2) for p in proj]
    dout = torch.randn(B, L, H * d, generator=g).to(torch.bfloat16).cuda().view(B, L, H, d).transpose(1, 2)
    out, _ = mod(*views, None, mat)
    assert out.stride() == views[0].stride()
    out.backward(dout)
    grads = [p.grad.clone() for p in proj]
    cont = [v.detach().contiguous().requires_grad_() for v in views]
    out2, _ = mod(*cont, None, mat)
    out2.backward(dout.contiguous())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    for gp, c in zip(grads, cont):
        assert torch.equal(gp.view(B, L, H, d).transpose(1, 2), c.grad)


def test_bf16_rejects_element_patterns_and_fp32_handles():
    L, d, NB = 128, 32, 1
    sm, off, col = workloads.window_random_csr(L, 4, 12, seed=3)
    abi = BF16ABI(d, L, NB, 1)
    abi.set_pattern(sm, off, col)
    Q, K, V, dO = _bf16_inputs(NB, L, d, seed=4)
    with pytest.raises(_lib.SpionLibraryError, match="32x32 tiles"):
        abi.forward(Q, K, V)
    abi.close()
    fp32 = SparseABI(d, L, NB, 32, with_mask=False)
    abi2 = BF16ABI(d, L, NB, 32)
    abi2.set_pattern(sm, off, col)
    good = abi2.handle
    abi2.handle = fp32.handle
    with pytest.raises(_lib.SpionLibraryError, match="bf16 init"):
        abi2.forward(Q, K, V)
    abi2.handle = good
    abi2.close()
    fp32.close()


def test_bf16_module_autograd_matches_dense_statement():
    B, H, L, d, bs = 2, 2, 256, 64, 64
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    mat = torch.from_numpy(_mask(L // bs, 0.5, seed=9)).cuda()
    g = torch.Generator().manual_seed(11)
    q, k, v, do = ((torch.randn(B, H, L, d, generator=g) * s).to(torch.bfloat16).cuda() for s in (1.0, 1.0, 1.0, 1.0))
    for t in (q, k, v):
        t.requires_grad_()
    mod = BlockAttentionBF16(cfg)
    out, zero = mod(q, k, v, torch.ones(B, L, device="cuda"), mat)
    assert zero == 0 and out.dtype == torch.bfloat16
    out.backward(do)
    qr, kr, vr = (t.detach().double().cpu().requires_grad_() for t in (q, k, v))
    pattern = mat.cpu().double().repeat_interleave(bs, 0).repeat_interleave(bs, 1)
    ref, _ = osa.dense_masked_attention(qr, kr, vr, pattern, None)
    ref.backward(do.double().cpu())
    assert_close_bf16(out.detach().float().cpu().numpy(), ref.detach().numpy(), "module out")
    for name, a, b in (("dq", q, qr), ("dk", k, kr), ("dv", v, vr)):
        assert_close_bf16(a.grad.float().cpu().numpy(), b.grad.numpy(), f"module {name}")


def test_bf16_scale_up_shape_agrees_with_fp32_path():
    """Config 5 at full size (B=4, H=8, L=16384, d=64, 64x64 blocks, band + global row/column + 1 % random):
    too large for the CPU oracle, so the bf16 kernels are compared with the fp32 tile kernels (themselves
    checked against the oracle at smaller sizes) on the same bf16-rounded inputs."""
    B, H, L, d, bs = 4, 8, 16384, 64, 64
    NB = B * H
    mat = workloads.config5_mask()
    from spion_amd.csr import block_mask_to_csr_host
    sm, off, col = block_mask_to_csr_host(mat, bs)
    g = torch.Generator().manual_seed(0)
    Q, K, V, dO = ((torch.randn(NB, L, d, generator=g) * s).to(torch.bfloat16).cuda() for s in (1.0, 1.0, 1.0, 1.0))
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    O, lse = abi.forward(Q, K, V)
    dQ, dK, dV = abi.backward(Q, K, V, O, lse, dO)
    torch.cuda.synchronize()
    ref = SparseABI(d, L, NB, bs, with_mask=False)
    ref.set_pattern(sm, off, col)
    Qf, Kf, Vf, dOf = (t.float() for t in (Q, K, V, dO))
    Or, P = ref.forward(Qf, Kf, Vf)
    dQr, dKr, dVr = ref.backward(Qf, Kf, Vf, P, dOf)
    torch.cuda.synchronize()
    del P
    for name, a, b in (("O", O, Or), ("dQ", dQ, dQr), ("dK", dK, dKr), ("dV", dV, dVr)):
        a = a.float()
        assert torch.isfinite(a).all(), name
        rel_l2 = ((a - b).pow(2).sum() / b.pow(2).sum()).sqrt().item()
        assert rel_l2 <= REL_TOL_BF16, f"{name}: relative L2 error {rel_l2:.3e}"
        tol = REL_TOL_BF16 * b.abs() + ROW_TOL_BF16 * b.pow(2).mean(-1, keepdim=True).sqrt() + REL_TOL_BF16 * b.pow(2).mean().sqrt()
        excess = ((a - b).abs() - tol).max().item()
        assert excess <= 0, f"{name}: exceeds the element tolerance by {excess}"
    abi.close()
    ref.close()


def test_bf16_scale_up_shape_matches_oracle_on_bounded_rows():
    """Config 5 at full size with the inputs of the benchmark (Q, K, V ~ N(0,1)/8, dO ~ N(0,1), rounded to bf16): the
    kernels run on all of it; the oracle, which cannot, restates a bounded part exactly.  It is given a pattern that
    keeps, for three heads, the complete rows of a few query strips -- the global block row (cut into chunks and
    merged), the first band strip, one from the middle, the last -- and of every strip that attends to two chosen key
    blocks.  O, the row statistic and dQ of those rows depend on nothing else, and neither do dK and dV of the two
    key blocks, whose contributing rows are all there.  (dK / dV of the global key block need every row; its chunked
    column strips are covered by the comparison with the fp32 kernels above and, against the oracle, at L = 2048.)"""
    B, H, L, d, bs = 4, 8, 16384, 64, 64
    NB, nb = B * H, L // bs
    mat = workloads.config5_mask()
    from spion_amd.csr import block_mask_to_csr_host
    sm, off, col = block_mask_to_csr_host(mat, bs)
    g = torch.Generator().manual_seed(0)
    Q, K, V, dO = ((torch.randn(NB, L, d, generator=g) * s).to(torch.bfloat16).cuda() for s in (0.125, 0.125, 0.125, 1.0))
    abi = BF16ABI(d, L, NB, bs)
    abi.set_pattern(sm, off, col)
    O, lse = abi.forward(Q, K, V)
    dQ, dK, dV = abi.backward(Q, K, V, O, lse, dO)
    torch.cuda.synchronize()

    heads = [0, 13, 31]
    key_blocks = [nb // 3, nb - 2]
    query_blocks = sorted({0, 1, nb // 2, nb - 1} | {int(i) for c in key_blocks for i in np.nonzero(mat[:, c])[0]})
    assert len(query_blocks) < 40, "the bounded part stays small"
    rows = np.concatenate([np.arange(i * bs, (i + 1) * bs) for i in query_blocks])
    sm_r = np.zeros_like(sm)
    sm_r[rows] = sm[rows]
    off_r = np.zeros(L + 1, dtype=off.dtype)
    np.cumsum(sm_r, out=off_r[1:])
    col_r = np.concatenate([col[off[r]:off[r + 1]] for r in rows]).astype(col.dtype)
    assert int(off_r[-1]) == col_r.size
    sel = lambda t: t[heads]
    ref = _oracle(sel(Q), sel(K), sel(V), sel(dO), sm_r, off_r, col_r)
    got_lse = sel(lse).cpu().numpy().astype(np.float64)[:, rows]
    assert np.max(np.abs(got_lse - ref["lse"][:, rows])) < 1e-3
    for name, t in (("O", O), ("dQ", dQ)):
        extra = ref["extra"][name][:, rows] if name in ref["extra"] else None
        assert_close_bf16(sel(t).float().cpu().numpy()[:, rows], ref[name][:, rows], f"config 5 rows {name}", extra=extra)
    keys = np.concatenate([np.arange(c * bs, (c + 1) * bs) for c in key_blocks])
    for name, t in (("dK", dK), ("dV", dV)):
        extra = ref["extra"][name][:, keys] if name in ref["extra"] else None
        assert_close_bf16(sel(t).float().cpu().numpy()[:, keys], ref[name][:, keys], f"config 5 key blocks {name}", extra=extra)
    abi.close()
