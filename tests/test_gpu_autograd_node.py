"""The compiled autograd node (spion_amd/csrc/autograd_node.cpp) against the Python function it mirrors
(spion_amd/attention_blockcuda.py, itself the counterpart of models/attention_blockcuda.py:20-112): both hand the same
tensors to the same entry points, so outputs, probabilities and gradients must agree bit for bit -- on contiguous
heads, on views of projections, on slices of a fused projection, with the key mask, and on an element pattern (whose
backward needs the dS scratch)."""
import numpy as np
import pytest
import torch

import spion_amd
from spion_amd import _lib, workloads
from spion_amd.attention import Attention

pytestmark = pytest.mark.gpu


def _module(B, H, L, d, bs, with_mask):
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    if with_mask:
        cpp = Attention._blockcuda_mask_compile_module()
        return spion_amd.CUDABlockMaskAttention(cfg, cpp, cpp.init(d, L, B * H, bs)), cpp
    cpp = Attention._blockcuda_compile_module()
    return spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs)), cpp


def _inputs(B, H, L, d, layout, seed):
    g = torch.Generator().manual_seed(seed)
    if layout == "contiguous":
        q, k, v = (torch.randn(B, H, L, d, generator=g).cuda() for _ in range(3))
    elif layout == "proj":  # [B, L, H*d] projections viewed as heads
        q, k, v = (torch.randn(B, L, H, d, generator=g).cuda().transpose(1, 2) for _ in range(3))
    else:  # slices of one [B, L, 3, H, d] projection
        buf = torch.randn(B, L, 3, H, d, generator=g).cuda()
        q, k, v = (buf[:, :, i].transpose(1, 2) for i in range(3))
    do = torch.randn(B, H, L, d, generator=g).cuda()
    return q, k, v, do


@pytest.mark.parametrize("layout", ["contiguous", "proj", "fused"])
@pytest.mark.parametrize("with_mask", [False, True])
@pytest.mark.parametrize("pattern", ["tile", "element"])
def test_node_equals_python_function(layout, with_mask, pattern):
    node = _lib.autograd_node()
    if node is None:
        pytest.skip("SPION_PY_NODE=1: the Python function is the only path in this process")
    B, H, L, d = 2, 2, 256, 32
    if pattern == "tile":
        bs = 32
        mat_np = workloads.band_random_block_mask(L // bs, 1, extra_frac=0.1, seed=3).astype(np.float32)
    else:
        bs = 1
        sm, off, col = workloads.window_random_csr(L, 40, 100, seed=3)
        mat_np = np.zeros((L, L), dtype=np.float32)
        mat_np[np.repeat(np.arange(L), sm), col] = 1.0
    mat = torch.from_numpy(mat_np).cuda()
    mod, cpp = _module(B, H, L, d, bs, with_mask)
    key_mask = workloads.valid_length_mask(B, L, L // 2, L, seed=5).cuda() if with_mask else torch.ones(B, L, device="cuda")
    results = []
    for use_node in (True, False):
        q, k, v, do = _inputs(B, H, L, d, layout, seed=11)  # the same values in fresh buffers of the same layout
        leaves = [q, k, v]
        for t in leaves:
            t.requires_grad_()
        if use_node:
            out, p = mod.run(*leaves, key_mask, mat)
        else:
            out, p = mod.attn_func.apply(*leaves, key_mask, mat, mod)
        gq, gk, gv = torch.autograd.grad(out, leaves, do)
        torch.cuda.synchronize()
        results.append((out.detach(), p.detach(), gq, gk, gv))
        if layout == "fused":  # the gradients come back as slices of one buffer in both cases
            assert _lib.adjacent_head_views(gq, gk, gv)
    for a, b, name in zip(results[0], results[1], ("out", "p", "dq", "dk", "dv")):
        assert a.shape == b.shape and a.stride() == b.stride(), name
        assert torch.equal(a, b), name
    cpp.destroy(mod.attn_handle)


def test_node_ignores_the_gradient_of_the_probabilities_and_reports_errors():
    node = _lib.autograd_node()
    if node is None:
        pytest.skip("SPION_PY_NODE=1")
    B, H, L, d, bs = 1, 2, 128, 32, 32
    mat = torch.from_numpy(workloads.band_random_block_mask(L // bs, 1, extra_frac=0.2, seed=1).astype(np.float32)).cuda()
    mod, cpp = _module(B, H, L, d, bs, False)
    ones = torch.ones(B, L, device="cuda")
    q, k, v, do = _inputs(B, H, L, d, "contiguous", seed=2)
    for t in (q, k, v):
        t.requires_grad_()
    out, p = mod(q, k, v, ones, mat)
    # only the probabilities are used downstream: their gradient is ignored, the inputs get the gradient of a zero dO
    (p.sum() + 0.0 * out.sum()).backward()
    assert torch.count_nonzero(q.grad) == 0 and torch.count_nonzero(k.grad) == 0 and torch.count_nonzero(v.grad) == 0
    with pytest.raises(ValueError):
        mod(q[:, :1], k[:, :1], v[:, :1], ones, mat)
    cpp.destroy(mod.attn_handle)
