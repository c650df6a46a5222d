"""Integration of the whole hot path in a 2-layer encoder training step (benchmark configuration 3 at reduced
size): dense phase -> score maps -> pattern discovery -> sparse phase forward/backward -> AdamW step, compared
with the same model whose attention layers are the CPU oracle in float64 (same weights, same batch)."""
import copy

import numpy as np
import pytest
import torch

import spion_amd
from oracle import pattern as op
from tests import encoder_harness as eh
from tests.abi_utils import assert_close

pytestmark = pytest.mark.gpu


def _copy_weights(src, dst):
    sd = {k: v.detach().cpu().double() for k, v in src.state_dict().items()}
    missing = dst.load_state_dict(sd, strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys


@pytest.mark.parametrize("key_mask", [False, True])
def test_encoder_step_matches_oracle_model(key_mask):
    torch.manual_seed(0)
    cfg = eh.model_config(L=256, batch=4, block_size=32, key_mask=key_mask, threshold=0.85)
    ids, mask, labels = eh.synthetic_batch(cfg, seed=1)
    model = eh.EncoderForSC(cfg, spion_amd.Attention).cuda()
    ref = eh.EncoderForSC(cfg, eh.OracleAttention).double()
    _copy_weights(model, ref)

    # ---- dense phase: losses and head/batch-averaged score maps
    loss_d, attn_lst = model(ids.cuda(), mask.cuda(), labels.cuda(), None, is_attn=True)
    loss_dr, attn_lst_r = ref(ids, mask.double(), labels, None, is_attn=True)
    assert_close(loss_d.detach().cpu().numpy(), loss_dr.detach().numpy(), what="dense-phase loss")
    for a, b in zip(attn_lst, attn_lst_r):
        assert a.shape == (cfg["max_seq_len"],) * 2
        assert_close(a.detach().cpu().numpy(), b.detach().numpy(), what="score map")

    # ---- pattern discovery on the GPU maps; bit-exact against the oracle walk on the same pooled maps
    mat_lst = spion_amd.generate_pattern_conv_ff(attn_lst, cfg)
    assert mat_lst.shape == (4, 2, 8, 8)
    maps = torch.stack([a.detach() for a in attn_lst])
    mats, pooled, thresh = spion_amd.discover_block_masks(maps, cfg["block_size"], mode="conv_ff",
                                                          threshold=cfg["threshold"], return_aux=True)
    for l in range(2):
        want = op.mask_from_pooled(pooled[l].cpu().numpy(), np.float32(thresh[l].item()))
        assert np.array_equal(mats[l].cpu().numpy().astype(np.int8), want)
        assert torch.equal(mat_lst[0][l], mats[l])

    # ---- switch both models to the sparse phase and take one optimizer step
    for layer in model.layers:
        layer.mha.reconstruct_for_blocksparse(cfg)
    opt, opt_r = eh.make_optimizer(model, lr=1e-3), eh.make_optimizer(ref, lr=1e-3)
    loss, _ = model(ids.cuda(), mask.cuda(), labels.cuda(), mat_lst)
    loss.mean().backward()
    mat_ref = mat_lst.cpu().double()
    loss_r, _ = ref(ids, mask.double(), labels, mat_ref)
    loss_r.mean().backward()
    assert_close(loss.detach().cpu().numpy(), loss_r.detach().numpy(), what="sparse-phase loss")
    grads = dict(model.named_parameters())
    for name, p_ref in ref.named_parameters():
        g = grads[name].grad
        assert g is not None, name
        assert_close(g.cpu().numpy(), p_ref.grad.numpy(), rel=2e-4, what=f"grad {name}")
    opt.step()
    opt_r.step()
    for (name, p), (_, p_ref) in zip(model.named_parameters(), ref.named_parameters()):
        assert_close(p.detach().cpu().numpy(), p_ref.detach().numpy(), what=f"weight after step {name}")
