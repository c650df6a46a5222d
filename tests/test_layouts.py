"""Host logic of the strided entry points: which [B, H, L, d] views the library is handed in place (CPU tensors:
only strides and addresses are looked at)."""
import torch

from spion_amd import _lib


def test_head_layout_of_projection_views():
    B, H, L, d = 2, 3, 64, 32
    proj = torch.zeros(B, L, H * d)
    v = proj.view(B, L, H, d).transpose(1, 2)
    lay = _lib.head_layout(v)
    assert (lay.batch_stride, lay.head_stride, lay.row_stride) == (L * H * d, d, H * d)
    c = torch.zeros(B, H, L, d)
    lay = _lib.head_layout(c)
    assert (lay.batch_stride, lay.head_stride, lay.row_stride) == (H * L * d, L * d, d)
    fused = torch.zeros(B, L, 3, H, d)
    q, k, v3 = (fused[:, :, i].transpose(1, 2) for i in range(3))
    lay = _lib.head_layout(k)
    assert (lay.batch_stride, lay.head_stride, lay.row_stride) == (L * 3 * H * d, d, 3 * H * d)
    assert _lib.adjacent_head_views(q, k, v3)


def test_head_layout_refuses_what_the_kernels_cannot_address():
    B, H, L, d = 1, 2, 32, 32
    assert _lib.head_layout(torch.zeros(B, H, L, d + 1)[..., :d]) is None        # row stride 33: not 16-byte rows
    assert _lib.head_layout(torch.zeros(B, H, L, d + 4)[..., 1:d + 1]) is None    # 4-byte offset
    assert _lib.head_layout(torch.zeros(B, H, L, 2 * d)[..., ::2]) is None        # last dimension strided
    assert _lib.head_layout(torch.zeros(B, H, d, L).transpose(2, 3)) is None      # feature-major
    ok = torch.zeros(B, H, L, d + 4)[..., :d]                                     # padded rows are fine
    assert _lib.head_layout(ok).row_stride == d + 4
    shared = torch.zeros(B, 1, L, d).expand(B, H, L, d)                           # one head shared by all: inputs only
    assert _lib.head_layout(shared).head_stride == 0
