"""The modules under HIP graph capture: a whole forward + backward step recorded once and replayed must give, on
every replay, bit for bit what the eager step gives -- with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import spion_amd
from spion_amd import workloads
from spion_amd.attention import Attention

pytestmark = pytest.mark.gpu


def _capture_step(module, args, q, k, v, do):
    """Warm up on a side stream (first calls analyse the pattern and allocate the library's workspaces, which a
    capture must not do), then record one step."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            for t in (q, k, v):
                t.grad = None
            out = module(q, k, v, *args)[0]
            out.backward(do)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for t in (q, k, v):
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = module(q, k, v, *args)[0]
        out.backward(do)
    return graph, out, [t.grad for t in (q, k, v)]  # the tensors every replay writes


def _eager_step(module, args, q, k, v, do):
    for t in (q, k, v):
        t.grad = None
    out = module(q, k, v, *args)[0]
    out.backward(do)
    return out.detach().clone(), [t.grad.clone() for t in (q, k, v)]


@pytest.mark.parametrize("kind", ["block", "blockmask", "dense", "bf16", "block_views", "blockmask_views", "dense_views",
                                  "bf16_views", "hybrid", "hybrid_views", "hybridmask_views", "global",
                                  "global_views"])
def test_whole_step_graph_replays_match_eager(kind):
    views = kind.endswith("_views")  # heads as views of [B, L, H*d] projections: the strided entry points
    kind = kind.split("_")[0]
    B, H, L, d, bs = 2, 2, 256, 32, 32
    hybrid = kind.startswith("hybrid")  # element-sparse pattern (window + scattered entries): seven launches a step
    if kind == "global":
        # a block row and a block column that span the sequence: every pass is two launches, the long strips on the
        # caller's stream and the others on the handle's side stream, forked and joined by events inside the capture
        L = 2048
        pattern = workloads.band_random_block_mask(L // bs, 1, extra_frac=0.05, seed=3)
        pattern[0, :] = 1.0
        pattern[:, 0] = 1.0
        mat = torch.from_numpy(pattern).cuda()
        kind = "block"
    elif hybrid:
        bs = 1
        sm, off, col = workloads.window_random_csr(L, 40, 100, seed=3)
        pattern = np.zeros((L, L), dtype=np.float32)
        pattern[np.repeat(np.arange(L), sm), col] = 1.0
        mat = torch.from_numpy(pattern).cuda()
        kind = "blockmask" if kind == "hybridmask" else "block"
    else:
        mat = torch.from_numpy(workloads.band_random_block_mask(L // bs, 1, extra_frac=0.1, seed=3)).cuda()
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    key_mask = torch.ones(B, L)
    key_mask[1, L - 56:] = 0
    key_mask = key_mask.cuda()
    if kind == "block":
        cpp = Attention._blockcuda_compile_module()
        module, args = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs)), (key_mask, mat)
    elif kind == "blockmask":
        cpp = Attention._blockcuda_mask_compile_module()
        module, args = spion_amd.CUDABlockMaskAttention(cfg, cpp, cpp.init(d, L, B * H, bs)), (key_mask, mat)
    elif kind == "dense":
        cpp = Attention._cuda_compile_module()
        module, args = spion_amd.CUDAAttention(cfg, cpp, cpp.init(d, L, B * H)), (key_mask,)
    else:
        module, args = spion_amd.BlockAttentionBF16(cfg), (key_mask, mat)
    dtype = torch.bfloat16 if kind == "bf16" else torch.float32
    q, k, v, do = (t.to(dtype) for t in workloads.qkv(B, H, L, d, seed=11, device="cuda"))
    if views:
        q, k, v, do = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v, do))
        assert module.reads_views and not q.is_contiguous()
    for t in (q, k, v):
        t.requires_grad_()
    ref_out, ref_grads = _eager_step(module, args, q, k, v, do)
    if hybrid:
        from spion_amd import _lib
        assert _lib.core().spion_last_path(module.attn_handle) == 3
    graph, out, static_grads = _capture_step(module, args, q, k, v, do)
    for replay in range(4):
        out.detach().zero_()
        for g in static_grads:
            g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref_out), f"{kind}: output of replay {replay} differs from the eager step"
        for name, g, r in zip("qkv", static_grads, ref_grads):
            assert torch.equal(g, r), f"{kind}: d{name} of replay {replay} differs from the eager step"
        # eager work of the same module (same handle, other buffers) between the replays
        e_out, e_grads = _eager_step(module, args, q, k, v, do)
        assert torch.equal(e_out, ref_out)
        for g, r in zip(e_grads, ref_grads):
            assert torch.equal(g, r)
    assert np.isfinite(ref_out.float().cpu().numpy()).all()


def test_long_strip_split_follows_the_callers_stream():
    """A pattern with a global block row and column (every pass: the long strips on the caller's stream, the others on
    the handle's side stream, joined by events): steps issued on torch's default stream and on two side streams in
    turn, without host synchronisation in between, give what the first step gave, bit for bit."""
    B, H, L, d, bs = 2, 2, 2048, 32, 32
    pattern = workloads.band_random_block_mask(L // bs, 1, extra_frac=0.05, seed=3)
    pattern[0, :] = 1.0
    pattern[:, 0] = 1.0
    mat = torch.from_numpy(pattern).cuda()
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    cpp = Attention._blockcuda_compile_module()
    module = spion_amd.CUDABlockAttention(cfg, cpp, cpp.init(d, L, B * H, bs))
    args = (torch.ones(B, L, device="cuda"), mat)
    q, k, v, do = workloads.qkv(B, H, L, d, seed=5, device="cuda")
    for t in (q, k, v):
        t.requires_grad_()
    ref_out, ref_grads = _eager_step(module, args, q, k, v, do)
    torch.cuda.synchronize()
    streams = [torch.cuda.current_stream(), torch.cuda.Stream(), torch.cuda.Stream()]
    results = []
    prev = streams[0]
    for i in range(6):
        s_ = streams[i % 3]
        s_.wait_stream(prev)  # the steps share the leaves' .grad and the handle's workspaces: one after the other
        with torch.cuda.stream(s_):
            results.append(_eager_step(module, args, q, k, v, do))
        prev = s_
    torch.cuda.current_stream().wait_stream(prev)
    torch.cuda.synchronize()
    for i, (out, grads) in enumerate(results):
        assert torch.equal(out, ref_out), f"step {i}: output differs"
        for name, g, r in zip("qkv", grads, ref_grads):
            assert torch.equal(g, r), f"step {i}: d{name} differs"
    cpp.destroy(module.attn_handle)


@pytest.mark.parametrize("sparse", [True, False])
def test_attention_layer_graph_replays_match_eager(sparse):
    """The whole ``Attention`` layer -- one GEMM for the three projections, heads read in place by the strided entry
    points, gradients handed back as slices of one buffer, output projection -- recorded once and replayed."""
    B, H, L, d, bs = 2, 2, 256, 32, 32
    cfg = dict(transformer_dim=H * d, head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs,
               task="lra-image", attention_dropout=0.0)
    torch.manual_seed(5)
    layer = Attention(cfg).cuda()
    mat = None
    if sparse:
        layer.reconstruct_for_blocksparse(cfg)
        mat = torch.from_numpy(workloads.band_random_block_mask(L // bs, 1, extra_frac=0.1, seed=3)).cuda()
    X = torch.randn(B, L, H * d, device="cuda", requires_grad=True)
    dY = torch.randn(B, L, H * d, device="cuda")
    key_mask = torch.ones(B, L, device="cuda")
    params = [X] + list(layer.parameters())

    def step():
        for t in params:
            t.grad = None
        y = layer(X, key_mask, mat)[0]
        y.backward(dY)
        return y

    # Every eager step ahead of the capture runs on a side stream and leaves no autograd graph behind.  A step on
    # the default stream whose output stays referenced keeps its AccumulateGrad nodes alive, and they belong to the
    # stream they were made on: the captured backward would then have to order the capturing stream against the
    # legacy default stream, which no capture may touch (torch warns of exactly this: "may ... break CUDA graph
    # capture if the AccumulateGrad node's stream is the default stream").  An earlier form of this test did that
    # and ended in a segmentation fault inside capture_end.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y = step()
        ref_y, ref_grads = y.detach().clone(), [t.grad.clone() for t in params]
        del y
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for t in params:
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = layer(X, key_mask, mat)[0]
        y_static.backward(dY)
    static_grads = [t.grad for t in params]
    for replay in range(3):
        y_static.detach().zero_()
        for g in static_grads:
            g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, ref_y), f"output of replay {replay} differs from the eager step"
        for i, (g, r) in enumerate(zip(static_grads, ref_grads)):
            assert torch.equal(g, r), f"gradient {i} of replay {replay} differs from the eager step"
        step()  # eager work on the same handle between the replays
        for t, r in zip(params, ref_grads):
            assert torch.equal(t.grad, r)
        for t, g in zip(params, static_grads):
            t.grad = g
