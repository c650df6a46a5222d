"""Pattern discovery: head-averaged attention maps -> layer-wise block masks, on the device.

The reference does this inline in its training drivers, on the host CPU: diagonal 31x31 filter,
block average pooling, a quantile threshold and the greedy path walk it calls flood fill
(main_conv_ff.py:35-62, :254-299), a top-k variant without the walk (main_conv.py:236-256) and a
pool-only variant (main_ff.py:253-272).  The functions here take the same inputs (the list of
per-layer score maps and the model config dict) and give the same ``mat_lst`` tensor
``[4, layers, nb, nb]`` of 0.0/1.0, computed by HIP kernels (spion_pattern_generate).
"""
from __future__ import annotations

import torch

from . import _lib

PATTERN_FLOOD = 0
PATTERN_TOPK = 1


def discover_block_masks(score_maps: torch.Tensor, block_size: int, *, mode: str = "conv_ff",
                         threshold: float | None = None, density: float | None = None,
                         ksize: int = 31, return_aux: bool = False):
    """score_maps [n, L, L] (fp32, on the GPU) -> block masks [n, nb, nb] float32 0/1.

    mode "conv_ff": filter + pool + quantile ``threshold`` + path walk   (main_conv_ff.py:254-278)
    mode "ff"     : pool + quantile ``threshold`` + path walk            (main_ff.py:253-272)
    mode "conv"   : filter + pool + top-k with ``density``               (main_conv.py:236-256)
    With ``return_aux`` also returns the pooled maps [n, nb, nb] and the thresholds [n].
    """
    if score_maps.dim() == 2:
        score_maps = score_maps.unsqueeze(0)
    if not score_maps.is_cuda:
        raise _lib.SpionLibraryError("pattern discovery runs on the GPU only; got a CPU tensor")
    x = score_maps.detach().to(torch.float32).contiguous()
    n, L, L2 = x.shape
    if L != L2 or L % block_size:
        raise ValueError(f"score maps must be square with L a multiple of block_size, got {tuple(x.shape)}")
    nb = L // block_size
    if mode == "conv_ff":
        k, kind, param = ksize, PATTERN_FLOOD, threshold
    elif mode == "ff":
        k, kind, param = 0, PATTERN_FLOOD, threshold
    elif mode == "conv":
        k, kind, param = ksize, PATTERN_TOPK, density
    else:
        raise ValueError(f"unknown mode {mode!r}")
    if param is None:
        raise ValueError("threshold (conv_ff / ff) or density (conv) is required")
    mat = torch.empty((n, nb, nb), dtype=torch.float32, device=x.device)
    pooled = torch.empty((n, nb, nb), dtype=torch.float32, device=x.device)
    thresh = torch.empty((n,), dtype=torch.float32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    rc = _lib.core().spion_pattern_generate(x.data_ptr(), n, L, block_size, k, kind, float(param),
                                            mat.data_ptr(), pooled.data_ptr(), thresh.data_ptr(), stream)
    if rc != 0:
        _lib.check_error("spion_pattern_generate")
        raise _lib.SpionLibraryError("spion_pattern_generate failed")
    return (mat, pooled, thresh) if return_aux else mat


def mean_score_map(attn: torch.Tensor) -> torch.Tensor:
    """attn [B, H, L, L] (fp32, on the GPU) -> [L, L], ``torch.mean(torch.mean(attn, dim=0), dim=0)``
    (models/model_transformer.py:136-137) in one pass of a HIP kernel.  Takes the permuted view the dense modules
    return (maps stored keys x queries) as it is, without a copy; any other layout is made contiguous first."""
    if attn.dim() != 4 or attn.shape[-1] != attn.shape[-2]:
        raise ValueError(f"expected [B, H, L, L], got {tuple(attn.shape)}")
    if not attn.is_cuda:
        raise _lib.SpionLibraryError("mean_score_map runs on the GPU only; got a CPU tensor")
    B, H, L, _ = attn.shape
    x = attn.detach()
    if x.dtype != torch.float32:
        x = x.float()
    key_major = x.stride() == (H * L * L, L * L, 1, L) and L > 1
    if not key_major:
        x = x.contiguous()
    out = torch.empty((L, L), dtype=torch.float32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    if _lib.core().spion_score_map_mean(x.data_ptr(), B, H, L, int(key_major), out.data_ptr(), stream) != 0:
        _lib.check_error("spion_score_map_mean")
        raise _lib.SpionLibraryError("spion_score_map_mean failed")
    return out


def _stack_layers(attn_lst, model_config):
    L = model_config["max_seq_len"]
    # the reference keeps the first L rows of each gathered map (main_conv_ff.py:255)
    return torch.stack([a[:L].detach() for a in attn_lst[: model_config["num_layers"]]], 0)


def _as_mat_lst(mats: torch.Tensor) -> torch.Tensor:
    # [layers, nb, nb] -> [4, layers, nb, nb]: one copy per data-parallel replica (main_conv_ff.py:298-299)
    return torch.stack([mats, mats, mats, mats], 0)


def generate_pattern_conv_ff(attn_lst, model_config) -> torch.Tensor:
    """SPION-CF masks for every layer; reads block_size, max_seq_len, num_layers, threshold."""
    mats = discover_block_masks(_stack_layers(attn_lst, model_config), model_config["block_size"],
                                mode="conv_ff", threshold=model_config["threshold"])
    return _as_mat_lst(mats)


def generate_pattern_ff(attn_lst, model_config) -> torch.Tensor:
    """SPION-F masks (no filter)."""
    mats = discover_block_masks(_stack_layers(attn_lst, model_config), model_config["block_size"],
                                mode="ff", threshold=model_config["threshold"])
    return _as_mat_lst(mats)


def generate_pattern_conv(attn_lst, model_config) -> torch.Tensor:
    """SPION-C masks (top-k of the pooled filtered map); reads density instead of threshold."""
    mats = discover_block_masks(_stack_layers(attn_lst, model_config), model_config["block_size"],
                                mode="conv", density=model_config["density"])
    return _as_mat_lst(mats)
