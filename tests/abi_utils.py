"""Test-side helpers: call the C ABI directly with torch device tensors and compare with the oracle."""
from __future__ import annotations

import numpy as np
import torch

from oracle import sparse_attention as osa
from spion_amd import _lib
from spion_amd.attention import Attention

REL_TOL_FP32 = 1e-4  # the tolerance the project states for fp32 results


def assert_close(got, ref, rel=REL_TOL_FP32, what=""):
    """|got - ref| <= rel * (|ref| + rms(ref)) element-wise (ref is the float64 oracle)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    err = np.abs(got - ref)
    tol = rel * (np.abs(ref) + rms)
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} outside tolerance; worst at {idx}: got {got[idx]!r}, "
            f"ref {ref[idx]!r}, err {err[idx]:.3e}, rms(ref) {rms:.3e}"
        )
    return float(err.max() / (rms + 1e-300))


class SparseABI:
    """One sparse-attention handle of a drop-in library, driven with raw pointers like the reference does."""

    def __init__(self, d, L, NB, block_size, with_mask, device="cuda"):
        self.lib = Attention._blockcuda_mask_compile_module() if with_mask else Attention._blockcuda_compile_module()
        self.with_mask = with_mask
        self.d, self.L, self.NB = d, L, NB
        self.dev = torch.device(device)
        self.handle = self.lib.init(d, L, NB, block_size)
        _lib.check_error("init")
        assert self.handle

    def close(self):
        if self.handle:
            self.lib.destroy(self.handle)
            self.handle = None

    def set_pattern(self, sum_mat, offsets, columns):
        self.sum_mat = torch.from_numpy(np.ascontiguousarray(sum_mat)).to(self.dev)
        self.offsets = torch.from_numpy(np.ascontiguousarray(offsets)).to(self.dev)
        cols = np.ascontiguousarray(columns) if len(columns) else np.zeros(1, np.int32)
        self.columns = torch.from_numpy(cols).to(self.dev)
        self.nnz = int(offsets[-1])

    def forward(self, Q, K, V, penalty=None):
        """Q, K, V: [NB, L, d] device tensors.  Returns (O [NB, L, d], P [NB, nnz])."""
        Kt = K.transpose(1, 2).contiguous()
        P = torch.full((self.NB * max(self.nnz, 1),), float("nan"), device=self.dev)
        O = torch.full((self.NB, self.L, self.d), float("nan"), device=self.dev)
        args = [self.handle, Q.data_ptr(), Kt.data_ptr(), V.data_ptr()]
        if self.with_mask:
            args.append(penalty.data_ptr())
        args += [P.data_ptr(), O.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(),
                 self.sum_mat.data_ptr(), self.nnz]
        self.lib.attn_forward(*args)
        _lib.check_error("attn_forward")
        return O, P[: self.NB * self.nnz].view(self.NB, self.nnz)

    def backward(self, Q, K, V, P, dO):
        Vt = V.transpose(1, 2).contiguous()
        n_tot = self.NB * max(self.nnz, 1)
        dP = torch.full((n_tot,), float("nan"), device=self.dev)
        dS = torch.full((n_tot,), float("nan"), device=self.dev)
        dQ, dK, dV = (torch.full((self.NB, self.L, self.d), float("nan"), device=self.dev) for _ in range(3))
        self.lib.attn_backward(self.handle, Q.data_ptr(), K.data_ptr(), Vt.data_ptr(), P.contiguous().data_ptr(),
                               dO.data_ptr(), dP.data_ptr(), dS.data_ptr(), dQ.data_ptr(), dK.data_ptr(),
                               dV.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(),
                               self.sum_mat.data_ptr(), self.nnz)
        _lib.check_error("attn_backward")
        return dQ, dK, dV

    def backward_with_out(self, Q, K, V, P, O, dO):
        """The library's own backward entry for callers that still hold the forward's output; no scratch."""
        Vt = V.transpose(1, 2).contiguous()
        dQ, dK, dV = (torch.full((self.NB, self.L, self.d), float("nan"), device=self.dev) for _ in range(3))
        _lib.core().spion_attn_backward_with_out(
            self.handle, Q.data_ptr(), K.data_ptr(), Vt.data_ptr(), P.contiguous().data_ptr(), O.data_ptr(),
            dO.data_ptr(), None, None, dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(), self.offsets.data_ptr(),
            self.columns.data_ptr(), self.sum_mat.data_ptr(), self.nnz)
        _lib.check_error("spion_attn_backward_with_out")
        return dQ, dK, dV

    def forward_rowmajor(self, Q, K, V, penalty=None):
        """The library's entry for row-major K (no transposed copy).  Returns (O, P)."""
        P = torch.full((self.NB * max(self.nnz, 1),), float("nan"), device=self.dev)
        O = torch.full((self.NB, self.L, self.d), float("nan"), device=self.dev)
        _lib.core().spion_attn_forward_rowmajor(
            self.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), penalty.data_ptr() if penalty is not None else None,
            P.data_ptr(), O.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(), self.sum_mat.data_ptr(),
            self.nnz)
        _lib.check_error("spion_attn_forward_rowmajor")
        return O, P[: self.NB * self.nnz].view(self.NB, self.nnz)

    def backward_rowmajor(self, Q, K, V, P, O, dO):
        """Row-major V, the forward's output handed over; dS scratch only where the element kernels need it."""
        dS = torch.full((self.NB * max(self.nnz, 1),), float("nan"), device=self.dev)
        dQ, dK, dV = (torch.full((self.NB, self.L, self.d), float("nan"), device=self.dev) for _ in range(3))
        _lib.core().spion_attn_backward_rowmajor(
            self.handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), P.contiguous().data_ptr(),
            O.data_ptr() if O is not None else None, dO.data_ptr(), dS.data_ptr(), dQ.data_ptr(), dK.data_ptr(),
            dV.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(), self.sum_mat.data_ptr(), self.nnz)
        _lib.check_error("spion_attn_backward_rowmajor")
        return dQ, dK, dV

    def forward_strided(self, q, k, v, out, penalty=None):
        """q, k, v, out: [B, H, L, d] views (any strides the library takes), read and written in place.  Returns P."""
        import ctypes
        P = torch.full((self.NB * max(self.nnz, 1),), float("nan"), device=self.dev)
        lin, lout = _lib.head_layout(q), _lib.head_layout(out)
        assert lin is not None and lout is not None
        assert k.stride() == q.stride() and v.stride() == q.stride()
        _lib.core().spion_attn_forward_strided(
            self.handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), penalty.data_ptr() if penalty is not None else None,
            P.data_ptr(), out.data_ptr(), self.offsets.data_ptr(), self.columns.data_ptr(), self.sum_mat.data_ptr(),
            self.nnz, q.shape[1], ctypes.addressof(lin), ctypes.addressof(lout))
        _lib.check_error("spion_attn_forward_strided")
        return P[: self.NB * self.nnz].view(self.NB, self.nnz)

    def backward_strided(self, q, k, v, P, out, dout, dq, dk, dv):
        import ctypes
        lin, lout, lgrad = _lib.head_layout(q), _lib.head_layout(out), _lib.head_layout(dq)
        assert lin is not None and lout is not None and lgrad is not None
        assert dout.stride() == out.stride() and dk.stride() == dq.stride() and dv.stride() == dq.stride()
        _lib.core().spion_attn_backward_strided(
            self.handle, q.data_ptr(), k.data_ptr(), v.data_ptr(), P.contiguous().data_ptr(), out.data_ptr(),
            dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), self.offsets.data_ptr(),
            self.columns.data_ptr(), self.sum_mat.data_ptr(), self.nnz, q.shape[1], ctypes.addressof(lin),
            ctypes.addressof(lout), ctypes.addressof(lgrad))
        _lib.check_error("spion_attn_backward_strided")

    def last_path(self):
        return _lib.core().spion_last_path(self.handle)

    def force_element(self, on=True):
        _lib.core().spion_force_element_path(self.handle, int(on))


def oracle_fwd_bwd(Q, K, V, dO, sum_mat, offsets, columns, penalty=None):
    """float64 oracle on numpy copies of the inputs.  Returns dict of O, P, dQ, dK, dV."""
    f = lambda t: t.detach().cpu().numpy().astype(np.float64)
    q, k, v, do = f(Q), f(K), f(V), f(dO)
    pen = None if penalty is None else penalty.detach().cpu().numpy().reshape(q.shape[0], -1).astype(np.float64)
    O, P = osa.csr_attention_forward(q, k, v, offsets, columns, sum_mat, pen)
    dQ, dK, dV, _ = osa.csr_attention_backward(q, k, v, P, do, offsets, columns)
    return dict(O=O, P=P, dQ=dQ, dK=dK, dV=dV)


def run_and_check(abi: SparseABI, Q, K, V, dO, penalty=None, rel=REL_TOL_FP32, tag=""):
    """Forward + backward through the ABI, compared with the oracle.  Returns the GPU results."""
    ref = oracle_fwd_bwd(Q, K, V, dO, abi.sum_mat.cpu().numpy(), abi.offsets.cpu().numpy(),
                         abi.columns.cpu().numpy()[: abi.nnz], penalty)
    O, P = abi.forward(Q, K, V, penalty)
    dQ, dK, dV = abi.backward(Q, K, V, P, dO)
    torch.cuda.synchronize()
    got = dict(O=O, P=P, dQ=dQ, dK=dK, dV=dV)
    for name in ("P", "O", "dQ", "dK", "dV"):
        assert_close(got[name].cpu().numpy(), ref[name], rel, f"{tag} {name}")
    return got, ref
