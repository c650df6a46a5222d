"""The one-GEMM form of the layer's three projections (models/attention.py:84-86 with split_heads :136-139) against
three separate linear layers: values and every gradient, with the incoming gradients as separate tensors and as the
adjacent slices of one buffer the attention modules hand back (CPU, float64)."""
import pytest
import torch

from spion_amd import _lib
from spion_amd.attention import _FusedQKV


@pytest.mark.parametrize("adjacent", [False, True])
def test_fused_projection_matches_three_linear_layers(adjacent):
    torch.manual_seed(0)
    B, L, dim, H, d = 2, 16, 24, 2, 8
    X = torch.randn(B, L, dim, dtype=torch.float64, requires_grad=True)
    ws = [torch.randn(H * d, dim, dtype=torch.float64, requires_grad=True) for _ in range(3)]
    bs = [torch.randn(H * d, dtype=torch.float64, requires_grad=True) for _ in range(3)]
    q, k, v = _FusedQKV.apply(X, *ws, *bs, H, d)
    assert _lib.adjacent_head_views(q, k, v)
    if adjacent:
        buf = torch.randn(B, L, 3, H, d, dtype=torch.float64)
        grads = tuple(buf[:, :, i].transpose(1, 2) for i in range(3))
        assert _lib.adjacent_head_views(*grads)
    else:
        grads = tuple(torch.randn(B, H, L, d, dtype=torch.float64) for _ in range(3))
    torch.autograd.backward((q, k, v), grads)
    got = [X.grad.clone()] + [w.grad.clone() for w in ws] + [b.grad.clone() for b in bs]
    for t in [X] + ws + bs:
        t.grad = None
    split = lambda y: y.view(B, L, H, d).transpose(1, 2)
    ref_out = [split(torch.nn.functional.linear(X, w, b)) for w, b in zip(ws, bs)]
    for a, b in zip((q, k, v), ref_out):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)
    torch.autograd.backward(ref_out, grads)
    for a, b in zip(got, [X.grad] + [w.grad for w in ws] + [b.grad for b in bs]):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_adjacent_heads_helpers():
    q, k, v = _lib.empty_adjacent_heads(2, 2, 64, 32, "cpu")
    assert q.shape == (2, 2, 64, 32) and _lib.adjacent_head_views(q, k, v)
    assert not _lib.adjacent_head_views(k, q, v)
    assert not _lib.adjacent_head_views(q.contiguous(), k.contiguous(), v.contiguous())
