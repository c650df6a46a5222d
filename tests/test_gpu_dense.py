"""Parity of the dense-phase HIP kernels with the float64 oracle, through the C ABI (GPU box only)."""
import numpy as np
import pytest
import torch

from oracle import dense_attention as oda
from oracle import sparse_attention as osa
from spion_amd import _lib, workloads
from spion_amd.attention import Attention
from tests.abi_utils import assert_close

pytestmark = pytest.mark.gpu


def _run_dense(d, L, NB, Q, K, V, dO, pen=None, moved_map=False):
    """Drive attn.so / attn_mask.so with the reference's operand layouts (models/attention_cuda.py:18-74).
    ``moved_map``: hand the backward a copy of the map at another address, so that it cannot use the copy of Out
    the forward filed under the original one and must sweep the map for its row sums."""
    lib = Attention._cuda_mask_compile_module() if pen is not None else Attention._cuda_compile_module()
    h = lib.init(d, L, NB)
    _lib.check_error("init")
    nan = float("nan")
    Qt, Kt, Vt, dOt = (t.transpose(1, 2).contiguous() for t in (Q, K, V, dO))
    attn = torch.full((NB, L, L), nan, device="cuda")
    out_t = torch.full((NB, d, L), nan, device="cuda")
    args = [h, Qt.data_ptr(), K.data_ptr(), Vt.data_ptr()]
    if pen is not None:
        args.append(pen.data_ptr())
    lib.attn_forward(*args, attn.data_ptr(), out_t.data_ptr())
    _lib.check_error("attn_forward")
    dq, dk, dv = (torch.full((NB, d, L), nan, device="cuda") for _ in range(3))
    if moved_map:
        attn = attn.clone()
    lib.attn_backward(h, Qt.data_ptr(), Kt.data_ptr(), V.data_ptr(), attn.data_ptr(), dOt.data_ptr(), None, None,
                      None, dq.data_ptr(), dk.data_ptr(), dv.data_ptr())
    _lib.check_error("attn_backward")
    torch.cuda.synchronize()
    lib.destroy(h)
    tr = lambda t: t.transpose(1, 2).cpu().numpy()
    return dict(O=tr(out_t), P=tr(attn), dQ=tr(dq), dK=tr(dk), dV=tr(dv))


@pytest.mark.parametrize("L,d,NB,with_mask", [(128, 32, 3, False), (256, 64, 2, False), (256, 32, 4, True),
                                              (1024, 32, 2, False), (96, 32, 2, False), (160, 32, 4, True),
                                              (992, 32, 2, False), (1024, 32, 4, True), (1056, 32, 2, False), (1088, 32, 4, True), (2048, 32, 2, False)])
def test_dense_matches_oracle(L, d, NB, with_mask):
    g = torch.Generator().manual_seed(L + d)
    Q, K, V, dO = (torch.randn(NB, L, d, generator=g).cuda() for _ in range(4))
    pen = None
    pen_np = None
    if with_mask:
        km = np.ones((NB // 2, L), np.float32)
        km[0, 130:] = 0
        km[1, 33:] = 0
        pen_np = osa.key_penalty_from_mask(km, 2)
        pen = torch.from_numpy(pen_np).cuda()
    got = _run_dense(d, L, NB, Q, K, V, dO, pen)
    f = lambda t: t.cpu().numpy().astype(np.float64)
    O, P = oda.dense_attention_forward(f(Q), f(K), f(V), None if pen_np is None else pen_np.astype(np.float64))
    dQ, dK, dV = oda.dense_attention_backward(f(Q), f(K), f(V), P, f(dO))
    for name, ref in (("P", P), ("O", O), ("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(got[name], ref, what=f"dense L={L} d={d} {name}")
    assert_close(got["P"].sum(-1), np.ones((NB, L)), what="rows of P sum to one")
    if with_mask:
        assert (got["P"][0][:, 130:] == 0).all() and (got["P"][2][:, 33:] == 0).all()


def _views(B, H, L, d, layout, n, seed, fill=None):
    """n tensors seen as [B, H, L, d]: "plain" contiguous, "proj" each a [B, L, H*d] projection, "fused" slices of
    one [B, L, n, H, d+4] buffer."""
    g = torch.Generator().manual_seed(seed)
    if layout == "plain":
        bufs = [torch.randn(B, H, L, d, generator=g).cuda() for _ in range(n)]
        views = bufs
    elif layout == "proj":
        bufs = [torch.randn(B, L, H * d, generator=g).cuda() for _ in range(n)]
        views = [b.view(B, L, H, d).transpose(1, 2) for b in bufs]
    else:
        buf = torch.randn(B, L, n, H, d + 4, generator=g).cuda()
        bufs = [buf]
        views = [buf[:, :, i, :, :d].transpose(1, 2) for i in range(n)]
    if fill is not None:
        for b in bufs:
            b.fill_(fill)
    return bufs, views


@pytest.mark.parametrize("layout,L,with_mask,d", [
    ("plain", 256, False, 32), ("proj", 256, True, 32), ("fused", 160, False, 32), ("proj", 1024, False, 32),
    ("proj", 1088, True, 32), ("fused", 2048, False, 32),
    ("plain", 256, False, 64), ("proj", 288, True, 64), ("fused", 160, False, 64), ("proj", 1024, True, 64),
    ("fused", 32, False, 64), ("proj", 2048, False, 64), ("plain", 1056, True, 64)])
def test_dense_strided_entry_points(layout, L, with_mask, d):
    """spion_dense_forward_strided / spion_dense_backward_strided: row-major heads, possibly interleaved in the
    memory of [B, L, H*d] projections, against the oracle and -- d = 32, where both entries run the same kernels --
    bit for bit against the reference's ABI on transposed copies of the same tensors (d = 64: to rounding)."""
    import ctypes
    B, H = 2, 2
    NB = B * H
    lib = Attention._cuda_mask_compile_module() if with_mask else Attention._cuda_compile_module()
    h = lib.init(d, L, NB)
    _lib.check_error("init")
    _, (q, k, v) = _views(B, H, L, d, layout, 3, seed=L)
    _, (dout,) = _views(B, H, L, d, "plain" if layout == "plain" else "proj", 1, seed=L + 1)
    _, (out,) = _views(B, H, L, d, "plain" if layout == "plain" else "proj", 1, seed=0, fill=float("nan"))
    gbufs, (dq, dk, dv) = _views(B, H, L, d, layout, 3, seed=0, fill=-7.0)
    pen = pen_np = None
    if with_mask:
        km = np.ones((B, L), np.float32)
        km[0, 130:] = 0
        km[1, 33:] = 0
        pen_np = osa.key_penalty_from_mask(km, H)
        pen = torch.from_numpy(pen_np).cuda()
    attn = torch.full((NB, L, L), float("nan"), device="cuda")
    lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
    A = ctypes.addressof
    core = _lib.core()
    core.spion_dense_forward_strided(h, q.data_ptr(), k.data_ptr(), v.data_ptr(), pen.data_ptr() if with_mask else None,
                                     attn.data_ptr(), out.data_ptr(), H, A(lin), A(lout))
    _lib.check_error("dense forward strided")
    core.spion_dense_backward_strided(h, q.data_ptr(), k.data_ptr(), v.data_ptr(), attn.data_ptr(), out.data_ptr(),
                                      dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), H, A(lin), A(lout),
                                      A(lgrad))
    _lib.check_error("dense backward strided")
    torch.cuda.synchronize()
    lib.destroy(h)
    flat = lambda t: t.reshape(NB, L, d).contiguous()
    Q, K, V, dO = flat(q), flat(k), flat(v), flat(dout)
    abi = _run_dense(d, L, NB, Q, K, V, dO, pen)
    got = dict(O=flat(out).cpu().numpy(), P=attn.transpose(1, 2).cpu().numpy(), dQ=flat(dq).cpu().numpy(),
               dK=flat(dk).cpu().numpy(), dV=flat(dv).cpu().numpy())
    for name in ("P", "O", "dQ", "dK", "dV"):
        if d == 32:
            assert np.array_equal(got[name], abi[name]), f"{name}: differs from the reference ABI's result"
        else:
            assert_close(got[name], abi[name].astype(np.float64), what=f"dense strided d=64 vs reference ABI: {name}")
    if layout == "fused":
        assert (gbufs[0][..., d:] == -7.0).all(), "padding between the heads' rows was written"
    if L <= 1088:
        f = lambda t: t.cpu().numpy().astype(np.float64)
        O, P = oda.dense_attention_forward(f(Q), f(K), f(V), None if pen_np is None else pen_np.astype(np.float64))
        gQ, gK, gV = oda.dense_attention_backward(f(Q), f(K), f(V), P, f(dO))
        for name, ref in (("P", P), ("O", O), ("dQ", gQ), ("dK", gK), ("dV", gV)):
            assert_close(got[name], ref, what=f"dense strided {layout} L={L} {name}")


def test_dense_backward_without_the_kept_output():
    L, d, NB = 256, 32, 2
    g = torch.Generator().manual_seed(5)
    Q, K, V, dO = (torch.randn(NB, L, d, generator=g).cuda() for _ in range(4))
    got = _run_dense(d, L, NB, Q, K, V, dO, moved_map=True)
    f = lambda t: t.cpu().numpy().astype(np.float64)
    O, P = oda.dense_attention_forward(f(Q), f(K), f(V), None)
    dQ, dK, dV = oda.dense_attention_backward(f(Q), f(K), f(V), P, f(dO))
    for name, ref in (("dQ", dQ), ("dK", dK), ("dV", dV)):
        assert_close(got[name], ref, what=f"dense, map at another address: {name}")


@pytest.mark.parametrize("with_mask,d,L", [(False, 32, 128), (True, 32, 128), (True, 64, 192), (False, 64, 2080)])
def test_dense_modules_autograd(with_mask, d, L):
    """The dense modules against float64 autograd; d = 64 takes the row-major entry points up to L = 2048 and the
    reference's ABI beyond."""
    import spion_amd

    B, H = 2, 2
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=32)
    if with_mask:
        cpp = Attention._cuda_mask_compile_module()
        mod = spion_amd.CUDAMaskAttention(cfg, cpp, cpp.init(d, L, B * H))
    else:
        cpp = Attention._cuda_compile_module()
        mod = spion_amd.CUDAAttention(cfg, cpp, cpp.init(d, L, B * H))
    q, k, v, do = workloads.qkv(B, H, L, d, seed=7, device="cuda")
    key_mask = torch.ones(B, L)
    if with_mask:
        key_mask[1, 90:] = 0
    for t in (q, k, v):
        t.requires_grad_()
    out, attn = mod(q, k, v, key_mask.cuda())
    assert out.shape == (B, H, L, d) and attn.shape == (B, H, L, L)
    out.backward(do)
    qc, kc, vc = (t.detach().double().cpu().requires_grad_() for t in (q, k, v))
    s = qc @ kc.transpose(-1, -2) * float(np.float32(1.0) / np.sqrt(np.float32(d)))
    if with_mask:
        s = s - 1e6 * (1 - key_mask.double())[:, None, None, :]
    p = torch.softmax(s, -1)
    o = p @ vc
    o.backward(do.double().cpu())
    assert_close(out.detach().cpu().numpy(), o.detach().numpy(), what="dense module out")
    assert_close(attn.detach().cpu().numpy(), p.detach().numpy(), what="dense module attn")
    for name, a, b in (("dq", q, qc), ("dk", k, kc), ("dv", v, vc)):
        assert_close(a.grad.cpu().numpy(), b.grad.numpy(), what=f"dense module {name}")


def test_dense_strided_limits_at_head_dimension_64():
    """Head dimension 64: the row-major forward refuses sequences beyond 2048 and the mean-emitting form, with a
    message and without touching the outputs; the module then goes through the reference's ABI."""
    import ctypes
    d, B, H, L = 64, 1, 2, 2080
    lib = Attention._cuda_compile_module()
    h = lib.init(d, L, B * H)
    _lib.check_error("init")
    q, k, v = (torch.zeros(B, H, L, d, device="cuda") for _ in range(3))
    out = torch.full((B, H, L, d), 3.0, device="cuda")
    attn = torch.full((2, 8), 5.0, device="cuda")  # never written
    lay = _lib.head_layout(q)
    A = ctypes.addressof(lay)
    core = _lib.core()
    core.spion_dense_forward_strided(h, q.data_ptr(), k.data_ptr(), v.data_ptr(), None, attn.data_ptr(),
                                     out.data_ptr(), H, A, A)
    with pytest.raises(_lib.SpionLibraryError, match="seq_len <= 2048"):
        _lib.check_error("dense forward strided")
    torch.cuda.synchronize()
    assert (out == 3.0).all() and (attn == 5.0).all()
    lib.destroy(h)
    import spion_amd
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=32)
    cpp = Attention._cuda_compile_module()
    mod = spion_amd.CUDAAttention(cfg, cpp, cpp.init(d, L, B * H))
    assert not mod.reads_views
