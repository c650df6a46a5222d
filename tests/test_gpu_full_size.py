"""Benchmark configurations 3 and 4, and configuration 5's shape in fp32, at their full sizes (GPU box only).

The float64 oracle cannot run a whole batch of these sizes in seconds, so each case combines (a) the oracle on a
bounded part of the very tensors the full-size launch produced (two of the 64 heads; four of the 256 samples) with
(b) properties that hold at any size: finite results, rows of P summing to less than one, exact zeros on padded
keys, linearity of the backward in dO.  Tolerance: 1e-4 relative (tests/abi_utils.assert_close).
"""
import numpy as np
import pytest
import torch

import spion_amd
from oracle import sparse_attention as osa
from spion_amd import workloads
from tests import encoder_harness as eh
from tests.abi_utils import SparseABI, assert_close, oracle_fwd_bwd

pytestmark = pytest.mark.gpu


def test_config4_full_batch_properties():
    """Element-sparse CSR with key padding: B=32, H=2, L=4096, d=32, +-64 window plus random columns to 5 %."""
    B, H, L, d = 32, 2, 4096, 32
    NB = B * H
    sm, off, col = workloads.window_random_csr(L, 64, 205, seed=3)
    key_mask = workloads.valid_length_mask(B, L, 2048, 4096, seed=5)
    pen = torch.from_numpy(osa.key_penalty_from_mask(key_mask.numpy(), H)).cuda()
    q, k, v, do = workloads.qkv(B, H, L, d, seed=0, device="cuda")
    f = lambda t: t.reshape(NB, L, d).contiguous()
    Q, K, V, dO = f(q), f(k), f(v), f(do)
    abi = SparseABI(d, L, NB, 1, with_mask=True)
    abi.set_pattern(sm, off, col)
    O, P = abi.forward(Q, K, V, pen)
    dQ, dK, dV = abi.backward(Q, K, V, P, dO)
    torch.cuda.synchronize()
    assert abi.last_path() == 3   # window tiles on the MFMA units, random columns gathered
    # (a) the oracle on the first and the last head of the full-size launch
    for hsel in (0, NB - 1):
        s = slice(hsel, hsel + 1)
        ref = oracle_fwd_bwd(Q[s], K[s], V[s], dO[s], sm, off, col, penalty=pen[s])
        for name, got in (("O", O), ("P", P), ("dQ", dQ), ("dK", dK), ("dV", dV)):
            assert_close(got[s].cpu().numpy(), ref[name], what=f"config 4 head {hsel} {name}")
    # (b) finite; probabilities non-negative, rows sum to at most one; padded keys get exactly zero
    for t in (O, P, dQ, dK, dV):
        assert torch.isfinite(t).all()
    rows = torch.from_numpy(osa.csr_row_index(off)).cuda()
    rs = torch.zeros(NB, L, device="cuda").index_add_(1, rows, P)
    assert (P >= 0).all() and (rs <= 1 + 1e-5).all() and (rs > 0).all()
    cols = torch.from_numpy(col.astype(np.int64)).cuda()
    padded = pen.reshape(NB, L)[:, cols] > 0          # [NB, n]: entry sits on a padded key
    assert padded.any() and (P[padded] == 0).all()
    # gradients of padded keys vanish with their probabilities
    dead = pen.reshape(NB, L) > 0
    assert (dK[dead] == 0).all() and (dV[dead] == 0).all()
    # (c) the backward is linear in dO
    dQ2, dK2, dV2 = abi.backward(Q, K, V, P, 2.0 * dO)
    for a, b in ((dQ, dQ2), (dK, dK2), (dV, dV2)):
        assert torch.allclose(2.0 * a, b, rtol=1e-5, atol=1e-6)
    abi.close()


def test_config3_full_size_step_properties():
    """2-layer encoder training step at batch 256, L=1024 (d_model 64, FFN 128, H=2, d_head 32): dense phase,
    discovery, sparse forward + backward + AdamW at the full batch.  The float64 oracle model runs the first four
    samples; with a loss that weights only those samples the full-batch gradients must equal the oracle's."""
    torch.manual_seed(0)
    n_ref = 4
    cfg = eh.model_config(L=1024, batch=256, block_size=32, key_mask=False, threshold=0.90)
    ids, mask, labels = eh.synthetic_batch(cfg, seed=1)
    model = eh.EncoderForSC(cfg, spion_amd.Attention).cuda()
    with torch.no_grad():
        loss_d, attn_lst = model(ids.cuda(), mask.cuda(), labels.cuda(), None, is_attn=True)
    assert torch.isfinite(loss_d).all()
    mat_lst = spion_amd.generate_pattern_conv_ff(attn_lst, cfg)
    del attn_lst
    torch.cuda.empty_cache()
    dens = [float(m.mean()) for m in mat_lst[0]]
    assert all(0.03 < x < 0.5 for x in dens), dens
    for layer in model.layers:
        layer.mha.reconstruct_for_blocksparse(cfg)

    cfg_ref = dict(cfg, batch_size=n_ref)
    ref = eh.EncoderForSC(cfg_ref, eh.OracleAttention).double()
    ref.load_state_dict({k_: v_.detach().cpu().double() for k_, v_ in model.state_dict().items()}, strict=True)

    loss, _ = model(ids.cuda(), mask.cuda(), labels.cuda(), mat_lst)
    assert loss.shape == (256,) and torch.isfinite(loss).all()
    w = torch.zeros(256, device="cuda")
    w[:n_ref] = 1.0
    (loss * w).sum().backward()
    loss_r, _ = ref(ids[:n_ref], mask[:n_ref].double(), labels[:n_ref], mat_lst.cpu().double())
    loss_r.sum().backward()
    assert_close(loss[:n_ref].detach().cpu().numpy(), loss_r.detach().numpy(), what="config 3 loss of the first samples")
    grads = dict(model.named_parameters())
    for name, p_ref in ref.named_parameters():
        g = grads[name].grad
        assert g is not None and torch.isfinite(g).all(), name
        assert_close(g.cpu().numpy(), p_ref.grad.numpy(), rel=2e-4, what=f"config 3 grad {name}")

    # the whole batch: one optimizer step, finite everywhere, the weights move
    opt = eh.make_optimizer(model, lr=1e-3)
    opt.zero_grad(set_to_none=True)
    before = {n_: p_.detach().clone() for n_, p_ in model.named_parameters()}
    loss, _ = model(ids.cuda(), mask.cuda(), labels.cuda(), mat_lst)
    loss.mean().backward()
    g1 = {n_: p_.grad.clone() for n_, p_ in model.named_parameters()}
    # linearity of the backward in the output gradient, through both sparse layers
    opt.zero_grad(set_to_none=True)
    loss2, _ = model(ids.cuda(), mask.cuda(), labels.cuda(), mat_lst)
    (2.0 * loss2.mean()).backward()
    for n_, p_ in model.named_parameters():
        assert torch.isfinite(p_.grad).all(), n_
        assert torch.allclose(p_.grad, 2.0 * g1[n_], rtol=1e-4, atol=1e-7), n_
        p_.grad = g1[n_]
    opt.step()
    moved = 0
    for n_, p_ in model.named_parameters():
        assert torch.isfinite(p_).all(), n_
        moved += int(not torch.equal(p_, before[n_]))
    assert moved == len(before)


def test_config5_shape_in_fp32_matches_oracle_on_bounded_rows():
    """Configuration 5's shape (B=4, H=8, L=16384, d=64, 64x64 blocks, a global block row and column) through the fp32
    tile kernels at full size with the benchmark's inputs: every pass is two launches here (the global strips with
    eight wavefronts each, the others beside them).  The oracle restates a bounded part exactly, as in the bf16
    test of the same shape: for three heads, the complete rows of a few query strips -- the global block row, the
    first band strip, one from the middle, the last -- and of every strip that attends to two chosen key blocks.
    O, P and dQ of those rows depend on nothing else, and neither do dK and dV of the two key blocks."""
    from spion_amd.csr import block_mask_to_csr_host
    B, H, L, d, bs = 4, 8, 16384, 64, 64
    NB, nb = B * H, L // bs
    mat = workloads.config5_mask()
    sm, off, col = block_mask_to_csr_host(mat, bs)
    g = torch.Generator().manual_seed(0)
    Q, K, V, dO = ((torch.randn(NB, L, d, generator=g) * s).cuda() for s in (0.125, 0.125, 0.125, 1.0))
    abi = SparseABI(d, L, NB, bs, with_mask=False)
    abi.set_pattern(sm, off, col)
    O, P = abi.forward(Q, K, V)
    dQ, dK, dV = abi.backward(Q, K, V, P, dO)
    torch.cuda.synchronize()
    assert abi.last_path() == 1
    for t in (O, P, dQ, dK, dV):
        assert torch.isfinite(t).all()

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
    ref = oracle_fwd_bwd(sel(Q), sel(K), sel(V), sel(dO), sm_r, off_r, col_r)
    for name, t in (("O", O), ("dQ", dQ)):
        assert_close(sel(t).cpu().numpy()[:, rows], ref[name][:, rows], what=f"config 5 shape, fp32, rows: {name}")
    p_idx = np.concatenate([np.arange(off[r], off[r + 1]) for r in rows])
    assert_close(sel(P).cpu().numpy()[:, p_idx], ref["P"], what="config 5 shape, fp32, rows: P")
    keys = np.concatenate([np.arange(c * bs, (c + 1) * bs) for c in key_blocks])
    for name, t in (("dK", dK), ("dV", dV)):
        assert_close(sel(t).cpu().numpy()[:, keys], ref[name][:, keys], what=f"config 5 shape, fp32, key blocks: {name}")
    abi.close()
