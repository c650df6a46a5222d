"""Loading saved block masks into a model and the timed evaluation loop of the reference's inference driver.

* ``load_masks_for_inference`` does what main_inference.py:164-172 does -- read the pickled ``[4, layers, nb, nb]``
  mask tensor, switch every attention layer to its block-sparse module -- and, once per layer, what the reference
  repeats on every forward (models/attention_blockcuda.py:26-43): it builds the element-CSR index of the layer's
  mask on the host, uploads it and registers it with the layer's library handle from the host arrays
  (``spion_register_pattern``).  The library then holds the analysed pattern (tile index and its transpose) before
  the first batch arrives: no forward copies an index back or waits for the stream.
* ``timed_eval`` is the loop of main_inference.py:49-93: no-grad forward over the batches, mean loss and accuracy,
  total and per-step time from device events, peak memory.
"""
from __future__ import annotations

import time
from typing import Callable, Iterable

import torch

from .csr import block_mask_to_csr_host, index_from_host
from .masks import load_mask_list


def attach_mask_sidecars(attention_layers, mat_lst: torch.Tensor, config) -> list:
    """``attention_layers[l]`` (``spion_amd.Attention``) gets its block module (if it has none yet) and the prebuilt,
    registered index of ``mat_lst[0][l]``.  Returns the indices (one ``CsrIndex`` per layer)."""
    if mat_lst.dim() != 4 or mat_lst.shape[1] != len(attention_layers):
        raise ValueError(f"mask tensor {tuple(mat_lst.shape)} does not match {len(attention_layers)} layers")
    bs = int(config["block_size"])
    host = mat_lst[0].detach().cpu().numpy()
    out = []
    for l, layer in enumerate(attention_layers):
        if not hasattr(layer, "block_attn"):
            layer.reconstruct_for_blocksparse(config)
        mod = layer.block_attn
        mat = mat_lst[0][l]  # the very view Model.forward hands to the layer (models/model_transformer.py:139)
        sum_mat, offsets, columns = block_mask_to_csr_host(host[l], bs)
        idx = index_from_host(sum_mat, offsets, columns, mat.device, mod.attn_handle, keepalive=mat)
        mod.csr_cache.put(mat, bs, idx)
        out.append(idx)
    return out


def load_masks_for_inference(path: str, attention_layers, config, device) -> torch.Tensor:
    """Read a mask file written by either side, move it to ``device`` and prepare every layer for it."""
    mat_lst = load_mask_list(path, device=device)
    attach_mask_sidecars(attention_layers, mat_lst, config)
    return mat_lst


def timed_eval(step: Callable[[object], dict], batches: Iterable, device=None) -> dict:
    """Run ``step(batch)`` (which returns a dict with ``loss`` and ``accu`` tensors, as the reference's models do)
    over ``batches`` without gradients.  Returns mean loss, mean accuracy, step count, device time in ms (total and
    per step), host wall time in s and the peak of active device memory in MiB."""
    dev = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    losses, accs = [], []
    torch.cuda.reset_peak_memory_stats(dev)
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.time()
    start.record()
    with torch.no_grad():
        for batch in batches:
            out = step(batch)
            losses.append(out["loss"].mean())
            accs.append(out["accu"].mean())
    end.record()
    torch.cuda.synchronize(dev)
    n = len(losses)
    if n == 0:
        raise ValueError("timed_eval: no batches")
    ms = start.elapsed_time(end)
    return {
        "loss": float(torch.stack(losses).mean()),
        "accu": float(torch.stack(accs).mean()),
        "steps": n,
        "total_ms": ms,
        "ms_per_step": ms / n,
        "wall_s": time.time() - t0,
        "peak_active_mib": torch.cuda.memory_stats(dev).get("active_bytes.all.peak", 0) >> 20,
    }
