"""Pattern discovery kernels vs the oracle: pooled maps to 1 ulp-level, masks bit-exact (GPU box only)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import pattern as op
from spion_amd import discover_block_masks, generate_pattern_conv, generate_pattern_conv_ff, generate_pattern_ff
from spion_amd import workloads

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _check_maps(maps, bs, q, ksize):
    """GPU masks against (1) the oracle's walk on the GPU's own pooled map (always) and (2) the mask of the
    independent float64 route, whenever every decision of that route's walk is further from flipping than eight
    times the difference between the two pooled maps (or the maps are bit-identical).  At least one map of every
    call must take the second comparison: a call whose maps all sit on a near-tie fails instead of passing unseen."""
    mode = "conv_ff" if ksize else "ff"
    mat, pooled, thresh = discover_block_masks(maps.cuda(), bs, mode=mode, threshold=q, ksize=ksize or 31,
                                               return_aux=True)
    mat, pooled, thresh = mat.cpu().numpy(), pooled.cpu().numpy(), thresh.cpu().numpy()
    independent = 0
    for i in range(maps.shape[0]):
        ref_mask, ref_pooled, ref_thresh = op.generate_mask_conv_ff(maps[i].numpy(), bs, q, ksize=ksize, route="fp64")
        # fp64 accumulation on both sides, one rounding: equal except for double-rounding ties
        assert np.max(np.abs(pooled[i] - ref_pooled) / np.abs(ref_pooled).max()) < 2e-7
        # the walk is checked on the GPU's own pooled map: bit-exact by construction of the oracle
        t_gpu = op.quantile_linear(pooled[i], q)[0]
        assert abs(float(thresh[i]) - float(t_gpu)) <= np.spacing(np.float32(abs(t_gpu)))
        assert np.array_equal(mat[i].astype(np.int8), op.mask_from_pooled(pooled[i], np.float32(thresh[i])))
        nz = ref_pooled != 0
        err = float(np.max(np.abs(pooled[i][nz].astype(np.float64) - ref_pooled[nz]) / np.abs(ref_pooled[nz]))) if nz.any() else 0.0
        margin = op.decision_margin(ref_pooled, q)
        if np.array_equal(pooled[i], ref_pooled) or margin > 8 * err:
            independent += 1
            assert np.array_equal(mat[i].astype(np.int8), ref_mask), (i, margin, err)
    assert independent > 0, "no map of this case could be compared with the independent float64 route"
    return mat, pooled, thresh


@pytest.mark.parametrize("L,bs,q,ksize", [(256, 32, 0.9, 31), (512, 64, 0.96, 31), (256, 16, 0.75, 31),
                                          (256, 32, 0.9, 0), (128, 32, 0.5, 7)])
def test_pattern_small_maps(L, bs, q, ksize):
    g = torch.Generator().manual_seed(L + bs)
    maps = torch.softmax(torch.randn(3, L, L, generator=g) * 2, -1)
    maps[1] += 0.02 * torch.eye(L)
    _check_maps(maps, bs, q, ksize)


@pytest.mark.parametrize("L,bs", [(4096, 32), (6400, 32)])
def test_pattern_large_block_grids(L, bs):
    """Block grids of 128 x 128 (pooled map walked from LDS) and 200 x 200 (walked from global memory)."""
    g = torch.Generator().manual_seed(L)
    maps = torch.rand(1, L, L, generator=g)
    maps = maps / maps.sum(-1, keepdim=True)
    maps[0] += (2.0 / L) * torch.eye(L)
    _check_maps(maps, bs, 0.95, 31)


def test_pattern_config2_bit_exact_against_both_routes():
    """Config 2: two 1024x1024 maps, 31x31 diagonal filter, 32x32 pooling, q = 0.90.
    The seed is one whose decision margin exceeds the float32-route error (tests/golden/config2.json),
    so the reference's float32 PyTorch route, the float64 route and the GPU must give the same masks."""
    meta = json.load(open(os.path.join(GOLDEN, "config2.json")))
    maps = workloads.score_maps_config2(2, 1024, 32, seed=meta["seed"])
    mat, pooled, thresh = _check_maps(maps, 32, 0.90, 31)
    golden = np.load(os.path.join(GOLDEN, "config2_masks.npy"))
    assert np.array_equal(mat.astype(np.int8), golden)
    for i in range(2):
        m32, _, _ = op.generate_mask_conv_ff(maps[i].numpy(), 32, 0.90, route="torch")
        assert np.array_equal(mat[i].astype(np.int8), m32)


@pytest.mark.parametrize("which", [0, 1, 2])
def test_pattern_config2_more_seeded_maps_bit_exact(which):
    """Three more seeded pairs of configuration-2 maps (the next largest decision margins of the scan that chose the
    fixture's seed, 4e-4 and more against a float32-route difference of 2e-6): the GPU masks equal the committed
    ones and those of both oracle routes."""
    meta = json.load(open(os.path.join(GOLDEN, "config2.json")))["more"][which]
    maps = workloads.score_maps_config2(2, 1024, 32, seed=meta["seed"])
    mat, _, _ = _check_maps(maps, 32, 0.90, 31)
    golden = np.load(os.path.join(GOLDEN, "config2_more_masks.npy"))[which]
    assert np.array_equal(mat.astype(np.int8), golden)
    assert [int(m.sum()) for m in mat] == meta["blocks_set"]
    for i in range(2):
        m32, _, _ = op.generate_mask_conv_ff(maps[i].numpy(), 32, 0.90, route="torch")
        assert np.array_equal(mat[i].astype(np.int8), m32)


def test_discovery_repeats_on_any_stream_and_under_capture():
    """The result must not depend on how often, on which stream, or whether inside a graph the call is made.  The
    reference for every variant is the first eager call, itself checked against the oracle."""
    g = torch.Generator().manual_seed(5)
    maps = torch.softmax(torch.randn(5, 512, 512, generator=g) * 2, -1)
    ref_mat, ref_pooled, ref_thresh = _check_maps(maps, 32, 0.9, 31)
    dev_maps = maps.cuda()

    def same(out):
        mat, pooled, thresh = (t.cpu().numpy() for t in out)
        assert np.array_equal(mat, ref_mat) and np.array_equal(pooled, ref_pooled) and np.array_equal(thresh, ref_thresh)

    for _ in range(3):
        same(discover_block_masks(dev_maps, 32, mode="conv_ff", threshold=0.9, return_aux=True))
    for _ in range(2):  # two side streams
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                out = discover_block_masks(dev_maps, 32, mode="conv_ff", threshold=0.9, return_aux=True)
        side.synchronize()
        same(out)
    # recorded into a graph and replayed, with eager calls in between
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            out_g = discover_block_masks(dev_maps, 32, mode="conv_ff", threshold=0.9, return_aux=True)
    for _ in range(3):
        for t in out_g:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        same(out_g)
        same(discover_block_masks(dev_maps, 32, mode="conv_ff", threshold=0.9, return_aux=True))


@pytest.mark.parametrize("density", [0.2, 0.45, 0.8])
def test_pattern_topk_with_ties(density):
    """Maps of few exact levels (multiples of 1/4): pooled values are exact in both routes and tie massively, so
    the k-th largest value is shared by many blocks and the lower-flat-index rule decides."""
    L, bs = 512, 32
    g = torch.Generator().manual_seed(11)
    levels = torch.randint(0, 3, (2, L // 64, L // 64), generator=g).float() / 4
    maps = levels.repeat_interleave(64, 1).repeat_interleave(64, 2).contiguous()
    mat, pooled, _ = discover_block_masks(maps.cuda(), bs, mode="conv", density=density, return_aux=True)
    mat, pooled = mat.cpu().numpy(), pooled.cpu().numpy()
    for i in range(2):
        ref, ref_pooled, k = op.generate_mask_conv(maps[i].numpy(), bs, density)
        assert np.array_equal(pooled[i], ref_pooled)
        kth = np.sort(ref_pooled.ravel())[::-1][k - 1]
        assert (ref_pooled == kth).sum() > 1
        assert np.array_equal(mat[i].astype(np.int8), ref)


def test_pattern_topk_and_generators():
    L, bs = 256, 32
    g = torch.Generator().manual_seed(3)
    maps = torch.softmax(torch.randn(2, L, L, generator=g) * 2, -1)
    mat = discover_block_masks(maps.cuda(), bs, mode="conv", density=0.3).cpu().numpy()
    for i in range(2):
        ref, _, k = op.generate_mask_conv(maps[i].numpy(), bs, 0.3)
        assert np.array_equal(mat[i].astype(np.int8), ref)
    cfg = dict(max_seq_len=L, block_size=bs, num_layers=2, threshold=0.9, density=0.3)
    attn_lst = [torch.cat([m, m], 0).cuda() for m in maps]  # gathered maps carry extra rows; only the first L count
    for fn in (generate_pattern_conv_ff, generate_pattern_ff, generate_pattern_conv):
        ml = fn(attn_lst, cfg)
        assert ml.shape == (4, 2, L // bs, L // bs) and ml.dtype == torch.float32
        assert torch.equal(ml[0], ml[3]) and set(ml.unique().tolist()) <= {0.0, 1.0}
        assert (torch.diagonal(ml[0], dim1=-2, dim2=-1) == 1).all()


@pytest.mark.parametrize("B,H,L", [(3, 2, 64), (5, 3, 128), (64, 2, 1024)])
def test_mean_score_map_matches_torch(B, H, L):
    """Batch-then-head mean of the maps (models/model_transformer.py:136-137), for the key-major memory the dense
    modules hand out as a permuted view and for plain contiguous maps."""
    import spion_amd

    g = torch.Generator().manual_seed(B * L)
    base = torch.rand(B, H, L, L, generator=g).cuda()
    view = base.permute(0, 1, 3, 2)            # [B, H, Lq, Lk] over keys x queries memory
    for attn in (view, base):
        ref = torch.mean(torch.mean(attn.double(), dim=0), dim=0)
        got = spion_amd.mean_score_map(attn)
        assert got.shape == (L, L) and got.is_contiguous()
        assert torch.max(torch.abs(got.double() - ref)).item() < 1e-6
    # the view the dense module returns is taken without a copy
    cfg = dict(head_dim=32, num_head=H, max_seq_len=L, batch_size=B, block_size=32)
    if L <= 128:
        from spion_amd.attention import Attention
        cpp = Attention._cuda_compile_module()
        mod = spion_amd.CUDAAttention(cfg, cpp, cpp.init(32, L, B * H))
        q, k, v = (torch.randn(B, H, L, 32, generator=g).cuda() for _ in range(3))
        _, p = mod(q, k, v, torch.ones(B, L).cuda())
        assert p.stride() == (H * L * L, L * L, 1, L)
        ref = torch.mean(torch.mean(p.double(), dim=0), dim=0)
        assert torch.max(torch.abs(spion_amd.mean_score_map(p).double() - ref)).item() < 1e-6


@pytest.mark.parametrize("B,H,L,with_mask", [(3, 2, 64, False), (16, 2, 256, True), (64, 2, 1024, False), (4, 2, 2048, True),
                                                 (2, 2, 2080, False)])
def test_fused_score_map_from_the_dense_forward(B, H, L, with_mask):
    """The mean map the dense forward accumulates while it writes the maps (spion_dense_forward_strided_mean) against
    the two torch.mean passes of models/model_transformer.py:136-137 over the returned maps, in float64; outputs and
    maps of that forward agree with the plain forward's."""
    import spion_amd
    from spion_amd.attention import Attention

    d = 32
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=32)
    if with_mask:
        cpp = Attention._cuda_mask_compile_module()
        mod = spion_amd.CUDAMaskAttention(cfg, cpp, cpp.init(d, L, B * H))
    else:
        cpp = Attention._cuda_compile_module()
        mod = spion_amd.CUDAAttention(cfg, cpp, cpp.init(d, L, B * H))
    g = torch.Generator().manual_seed(B + L)
    q, k, v = (torch.randn(B, H, L, d, generator=g).cuda() for _ in range(3))
    lens = torch.randint(L // 2, L + 1, (B, 1), generator=g)
    key_mask = (torch.arange(L)[None, :] < lens).float().cuda()
    out0, p0 = mod(q, k, v, key_mask)
    assert mod.score_map is None
    mod.emit_score_map = True
    for rep in range(2):   # the second call reuses the partial maps the first one left
        out1, p1 = mod(q, k, v, key_mask)
        if L > 2048:   # the same two-sweep kernel with and without the mean
            assert torch.equal(out0, out1) and torch.equal(p0, p1)
        else:          # the logits stay in registers, split over wavefronts differently (mean beyond 1024: two sweeps)
            assert torch.allclose(out0, out1, rtol=1e-5, atol=1e-6) and torch.allclose(p0, p1, rtol=1e-5, atol=1e-9)
        ref = torch.mean(torch.mean(p1.double(), dim=0), dim=0)
        got = mod.score_map
        assert got.shape == (L, L) and got.is_contiguous()
        err = torch.max(torch.abs(got.double() - ref)).item()
        assert err < 2e-7 * max(1.0, float(ref.abs().max()) * 1e3), err
        assert torch.allclose(got.double(), ref, rtol=1e-5, atol=1e-9)
    # the map feeds discovery as it is
    m = spion_amd.discover_block_masks(mod.score_map[None], 32, mode="conv_ff", threshold=0.9)
    assert m.shape == (1, L // 32, L // 32)


def test_device_transition_detector_matches_host_detector():
    """spion_transition_update against the host statement of main_conv_ff.py:211-242 on the hand-worked sequences
    (1x1 maps: distances are absolute differences) and on random maps with a drift that settles."""
    from spion_amd import DeviceTransitionDetector, TransitionDetector

    def maps(*values):
        return [torch.tensor([[float(v)]]).cuda() for v in values]

    det = DeviceTransitionDetector(1)
    assert det.update(maps(0.0)) is False
    assert det.update(maps(10.0)) is False
    assert det.update(maps(10.5)) is True           # distance to the FIRST map 10.5: change 5 %
    assert det.update(maps(99.0)) is True
    det = DeviceTransitionDetector(1)
    det.update(maps(0.0)); det.update(maps(10.0))
    assert det.update(maps(20.0)) is False          # change 100 %: the kept map becomes 20
    assert det.update(maps(41.0)) is True           # distance 21: change 5 %
    for last, want in ((115.9, False), (114.99, True)):   # 15.9 % truncates to 15 (not below), 14.99 % to 14
        det = DeviceTransitionDetector(1)
        det.update(maps(0.0)); det.update(maps(100.0))
        assert det.update(maps(last)) is want
    det = DeviceTransitionDetector(2)
    det.update(maps(0.0, 0.0)); det.update(maps(10.0, 10.0))
    assert det.update(maps(10.5, 30.0)) is False    # layer 1 changed by 200 %
    assert abs(det.diff[0] - 5.0) < 1e-3 and abs(det.diff[1] - 200.0) < 1e-2

    # identical maps in a row: a previous distance of 0 never counts as settled (0/0, then 2/0)
    det = DeviceTransitionDetector(1)
    det.update(maps(5.0))
    assert det.update(maps(5.0)) is False
    assert det.update(maps(5.0)) is False
    assert det.update(maps(7.0)) is False
    assert det.update(maps(9.0)) is True

    # random maps: identical decisions and distances as the host detector, evaluation by evaluation
    g = torch.Generator().manual_seed(7)
    L, layers = 256, 3
    base = torch.rand(layers, L, L, generator=g)
    host, dev = TransitionDetector(layers), DeviceTransitionDetector(layers)
    decided = None
    for step in range(12):
        cur = base + torch.randn(layers, L, L, generator=g) * (0.5 / (1 + step) ** 2)
        a = host.update([cur[l] for l in range(layers)])
        b = dev.update(cur.cuda())
        assert a == b, step
        if host.before_distance:
            for x, y in zip(host.before_distance, dev.before_distance):
                assert abs(float(x) - y) <= 1e-5 * abs(float(x))
        if a and decided is None:
            decided = step
    assert decided is not None and decided >= 2
