"""Mask persistence and the inference path (GPU box only): masks written the way the reference writes them
(a plain pickle of the [4, layers, nb, nb] tensor as it lies on the GPU, main_conv_ff.py:298-306) are loaded into a
fresh model, every layer gets its prebuilt index registered with the library, and the timed evaluation loop of
main_inference.py:49-93 runs over a few batches; losses, accuracy and one backward are compared with the same
model on the float64 CPU oracle."""
import pickle

import numpy as np
import pytest
import torch

import spion_amd
from spion_amd import _lib
from tests import encoder_harness as eh
from tests.abi_utils import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("key_mask", [False, True])
def test_saved_masks_load_into_a_model_and_eval_loop_matches_oracle(tmp_path, key_mask):
    torch.manual_seed(3)
    cfg = eh.model_config(L=256, batch=4, block_size=32, key_mask=key_mask, threshold=0.85)
    trainer = eh.EncoderForSC(cfg, spion_amd.Attention).cuda()
    ids, mask, labels = eh.synthetic_batch(cfg, seed=2, device="cuda")
    with torch.no_grad():
        _, attn_lst = trainer(ids, mask, labels, None, is_attn=True)
    mat_lst = spion_amd.generate_pattern_conv_ff(attn_lst, cfg)
    assert mat_lst.is_cuda and mat_lst.shape == (4, 2, 8, 8)
    path = str(tmp_path / "mat_lst_lra-image_test.pickle")
    with open(path, "wb") as f:   # the reference's own way of writing the file
        pickle.dump(mat_lst, f, pickle.HIGHEST_PROTOCOL)

    # a fresh model, as the inference driver builds it, with the trained weights
    model = eh.EncoderForSC(cfg, spion_amd.Attention).cuda()
    model.load_state_dict(trainer.state_dict())
    layers = [layer.mha for layer in model.layers]
    loaded = spion_amd.load_masks_for_inference(path, layers, cfg, "cuda")
    assert torch.equal(loaded, mat_lst)
    core = _lib.core()
    for layer in layers:
        h = layer.block_attn.attn_handle
        assert core.spion_debug_counter(h, 1) == 1 and core.spion_debug_counter(h, 0) == 0

    # evaluation loop over three batches
    batches = [eh.synthetic_batch(cfg, seed=10 + i, device="cuda") for i in range(3)]
    res = spion_amd.timed_eval(lambda b: model.outputs(b[0], b[1], b[2], loaded), batches)
    assert res["steps"] == 3 and res["total_ms"] > 0 and res["ms_per_step"] == res["total_ms"] / 3
    for layer in layers:   # the forwards found the registered analysis: nothing was copied back from the device
        h = layer.block_attn.attn_handle
        assert core.spion_debug_counter(h, 0) == 0 and core.spion_debug_counter(h, 1) == 1
        assert core.spion_last_path(h) == 1

    ref = eh.EncoderForSC(cfg, eh.OracleAttention).double()
    ref.load_state_dict({k_: v_.detach().cpu().double() for k_, v_ in trainer.state_dict().items()}, strict=True)
    mats_cpu = loaded.cpu().double()
    ref_loss, ref_acc = [], []
    with torch.no_grad():
        for b in batches:
            o = ref.outputs(b[0].cpu(), b[1].cpu().double(), b[2].cpu(), mats_cpu)
            ref_loss.append(o["loss"].mean())
            ref_acc.append(o["accu"].mean())
    assert abs(res["loss"] - float(torch.stack(ref_loss).mean())) <= 1e-4 * abs(float(torch.stack(ref_loss).mean()))
    assert res["accu"] == pytest.approx(float(torch.stack(ref_acc).mean()), abs=1e-6)

    # the loaded masks train as well: one backward through both layers against the oracle model
    loss, _ = model(*batches[0], loaded)
    loss.mean().backward()
    loss_r, _ = ref(batches[0][0].cpu(), batches[0][1].cpu().double(), batches[0][2].cpu(), mats_cpu)
    loss_r.mean().backward()
    grads = dict(model.named_parameters())
    for name, p_ref in ref.named_parameters():
        assert_close(grads[name].grad.cpu().numpy(), p_ref.grad.numpy(), rel=2e-4, what=f"grad {name}")


def test_mask_file_round_trip_both_ways(tmp_path):
    """Files written by save_mask_list are what the reference's loader (a plain pickle.load,
    main_inference.py:164-166) reads, and files the reference writes from CPU tensors load here."""
    m = spion_amd.stack_for_replicas([np.eye(4, dtype=np.float32), np.ones((4, 4), np.float32)])
    p1 = str(tmp_path / "a.pickle")
    spion_amd.save_mask_list(m.cuda(), p1)
    with open(p1, "rb") as f:
        back = pickle.load(f)   # our own file: written by this test, holds a plain tensor
    assert torch.equal(back, m)
    p2 = str(tmp_path / "b.pickle")
    with open(p2, "wb") as f:
        pickle.dump(m, f, pickle.HIGHEST_PROTOCOL)
    assert torch.equal(spion_amd.load_mask_list(p2), m)
    assert spion_amd.load_mask_list(p2, device="cuda").is_cuda
