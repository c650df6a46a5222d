"""spion_amd -- SPION layer-wise sparse attention for AMD MI355X (gfx950).

The package mirrors the reference's attention modules (models/attention*.py) on top of
hand-written HIP kernels reached through a C ABI (include/spion_hip.h) with ctypes.
There is no CPU or PyTorch fallback: every module raises if the built libraries are missing.
"""
from .attention import Attention, SoftmaxAttention, mask_task
from .attention_cuda import CUDAAttention
from .attention_cuda_mask import CUDAMaskAttention
from .attention_blockcuda import CUDABlockAttention
from .attention_blockcuda_mask import CUDABlockMaskAttention
from .attention_blockbf16 import BlockAttentionBF16
from .inference import attach_mask_sidecars, load_masks_for_inference, timed_eval
from .masks import DeviceTransitionDetector, TransitionDetector, load_mask_list, save_mask_list, stack_for_replicas
from .pattern import (
    discover_block_masks,
    generate_pattern_conv,
    generate_pattern_conv_ff,
    generate_pattern_ff,
    mean_score_map,
)

__all__ = [
    "Attention",
    "SoftmaxAttention",
    "mask_task",
    "CUDAAttention",
    "CUDAMaskAttention",
    "CUDABlockAttention",
    "CUDABlockMaskAttention",
    "BlockAttentionBF16",
    "attach_mask_sidecars",
    "load_masks_for_inference",
    "timed_eval",
    "TransitionDetector",
    "DeviceTransitionDetector",
    "load_mask_list",
    "save_mask_list",
    "stack_for_replicas",
    "discover_block_masks",
    "generate_pattern_conv",
    "generate_pattern_conv_ff",
    "generate_pattern_ff",
    "mean_score_map",
]
