"""ctypes loaders for the built HIP libraries (spion_amd/lib/*.so).

``libspion_hip.so`` carries the prefixed C ABI of include/spion_hip.h; ``attn.so``,
``attn_mask.so``, ``block_attn.so`` and ``block_attn_mask.so`` re-export one family each under the
un-prefixed names the reference binds (models/attention.py:141-191).  Loading fails loudly when a
library has not been built: there is no fallback path.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_int, c_void_p

import torch  # noqa: F401  (first: the HIP runtime PyTorch ships must be the one in the process)

LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")

_P = c_void_p
_cache: dict = {}


class SpionLibraryError(RuntimeError):
    pass


def lib_path(name: str) -> str:
    return os.path.join(LIB_DIR, name)


def _cdll(name: str) -> ctypes.CDLL:
    if name in _cache:
        return _cache[name]
    path = lib_path(name)
    if not os.path.exists(path):
        raise SpionLibraryError(
            f"{path} is missing: build the HIP libraries first (python -m spion_amd.build). "
            "spion_amd has no CPU fallback."
        )
    # default (local) symbol scope, as the reference loads its libraries: the drop-ins' generic names (init,
    # destroy, ...) stay out of the process-wide scope; they find libspion_hip.so through DT_NEEDED + $ORIGIN
    lib = ctypes.CDLL(path)
    _cache[name] = lib
    return lib


def autograd_node():
    """The compiled autograd node (lib/_spion_node.so, csrc/autograd_node.cpp), or None when SPION_PY_NODE=1 asks for
    the Python function instead (A/B timing, tests of the Python statement).  Both run the same kernels through the
    same entry points; a missing build is an error like any other missing library."""
    if "node" in _cache:
        return _cache["node"]
    mod = None
    if os.environ.get("SPION_PY_NODE", "0") != "1":
        import importlib.util

        path = lib_path("_spion_node.so")
        if not os.path.exists(path):
            raise SpionLibraryError(f"{path} is missing: build the libraries first (python -m spion_amd.build)")
        core()  # libspion_hip.so first: the node links against it
        spec = importlib.util.spec_from_file_location("_spion_node", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    _cache["node"] = mod
    return mod


def core() -> ctypes.CDLL:
    """libspion_hip.so with argtypes of the entry points that have no reference counterpart."""
    lib = _cdll("libspion_hip.so")
    if getattr(lib, "_spion_typed", False):
        return lib
    lib.spion_last_error.restype = c_char_p
    lib.spion_last_error.argtypes = []
    lib.spion_clear_error.argtypes = []
    lib.spion_clear_error.restype = None
    lib.spion_error_pending.argtypes = []
    lib.spion_error_pending.restype = c_int
    lib.spion_set_stream.argtypes = [_P, _P]
    lib.spion_set_stream.restype = None
    lib.spion_invalidate_pattern.argtypes = [_P]
    lib.spion_invalidate_pattern.restype = None
    lib.spion_forget_pattern.argtypes = [_P, _P, _P]
    lib.spion_forget_pattern.restype = None
    lib.spion_register_pattern.argtypes = [_P, _P, _P, c_int, _P, _P]
    lib.spion_register_pattern.restype = c_int
    lib.spion_handle_error.argtypes = [_P]
    lib.spion_handle_error.restype = c_char_p
    lib.spion_clear_handle_error.argtypes = [_P]
    lib.spion_clear_handle_error.restype = None
    lib.spion_last_path.argtypes = [_P]
    lib.spion_last_path.restype = c_int
    lib.spion_force_element_path.argtypes = [_P, c_int]
    lib.spion_force_element_path.restype = None
    lib.spion_set_backward_passes.argtypes = [_P, c_int]
    lib.spion_set_backward_passes.restype = None
    lib.spion_debug_counter.argtypes = [_P, c_int]
    lib.spion_debug_counter.restype = c_int
    lib.spion_use_output_cache.argtypes = [_P, c_int]
    lib.spion_use_output_cache.restype = None
    lib.spion_attn_backward_with_out.argtypes = [_P] * 15 + [c_int]
    lib.spion_attn_backward_with_out.restype = None
    lib.spion_attn_forward_rowmajor.argtypes = [_P] * 10 + [c_int]
    lib.spion_attn_forward_rowmajor.restype = None
    lib.spion_attn_backward_rowmajor.argtypes = [_P] * 14 + [c_int]
    lib.spion_attn_backward_rowmajor.restype = None
    lib.spion_attn_backward_noalloc.argtypes = [_P] * 13 + [c_int]
    lib.spion_attn_backward_noalloc.restype = None
    lib.spion_noalloc_max_rows.argtypes = []
    lib.spion_noalloc_max_rows.restype = ctypes.c_longlong
    lib.spion_attn_forward_strided.argtypes = [_P] * 10 + [c_int, c_int, _P, _P]
    lib.spion_attn_forward_strided.restype = None
    lib.spion_attn_backward_strided.argtypes = [_P] * 13 + [c_int, c_int, _P, _P, _P]
    lib.spion_attn_backward_strided.restype = None
    lib.spion_dense_forward_strided.argtypes = [_P] * 7 + [c_int, _P, _P]
    lib.spion_dense_forward_strided.restype = None
    lib.spion_dense_forward_strided_mean.argtypes = [_P] * 8 + [c_int, _P, _P]
    lib.spion_dense_forward_strided_mean.restype = None
    lib.spion_transition_update.argtypes = [_P, _P, c_int, ctypes.c_longlong, _P, _P, c_int, c_int, _P]
    lib.spion_transition_update.restype = c_int
    lib.spion_dense_backward_strided.argtypes = [_P] * 10 + [c_int, _P, _P, _P]
    lib.spion_dense_backward_strided.restype = None
    lib.spion_transpose_last2.argtypes = [_P, _P, c_int, c_int, c_int, _P]
    lib.spion_transpose_last2.restype = c_int
    lib.spion_version.restype = c_char_p
    lib.spion_version.argtypes = []
    lib.spion_pattern_generate.argtypes = [_P, c_int, c_int, c_int, c_int, c_int, c_double, _P, _P, _P, _P]
    lib.spion_pattern_generate.restype = c_int
    lib.spion_score_map_mean.argtypes = [_P, c_int, c_int, c_int, c_int, _P, _P]
    lib.spion_score_map_mean.restype = c_int
    for fam, extra in (("block", 0), ("blockmask", 1)):
        getattr(lib, f"spion_{fam}_init").argtypes = [c_int, c_int, c_int, c_int]
        getattr(lib, f"spion_{fam}_init").restype = _P
        getattr(lib, f"spion_{fam}_attn_forward").argtypes = [_P] * (9 + extra) + [c_int]
        getattr(lib, f"spion_{fam}_attn_forward").restype = None
        getattr(lib, f"spion_{fam}_attn_backward").argtypes = [_P] * 14 + [c_int]
        getattr(lib, f"spion_{fam}_attn_backward").restype = None
        getattr(lib, f"spion_{fam}_destroy").argtypes = [_P]
        getattr(lib, f"spion_{fam}_destroy").restype = None
    lib.spion_block_bf16_init.argtypes = [c_int, c_int, c_int, c_int]
    lib.spion_block_bf16_init.restype = _P
    lib.spion_block_bf16_attn_forward.argtypes = [_P] * 10 + [c_int]
    lib.spion_block_bf16_attn_forward.restype = None
    lib.spion_block_bf16_attn_backward.argtypes = [_P] * 14 + [c_int]
    lib.spion_block_bf16_attn_backward.restype = None
    lib.spion_block_bf16_attn_forward_strided.argtypes = [_P] * 10 + [c_int, c_int, _P, _P]
    lib.spion_block_bf16_attn_forward_strided.restype = None
    lib.spion_block_bf16_attn_backward_strided.argtypes = [_P] * 14 + [c_int, c_int, _P, _P, _P]
    lib.spion_block_bf16_attn_backward_strided.restype = None
    lib.spion_block_bf16_destroy.argtypes = [_P]
    lib.spion_block_bf16_destroy.restype = None
    for fam, extra in (("dense", 0), ("densemask", 1)):
        getattr(lib, f"spion_{fam}_init").argtypes = [c_int, c_int, c_int]
        getattr(lib, f"spion_{fam}_init").restype = _P
        getattr(lib, f"spion_{fam}_attn_forward").argtypes = [_P] * (6 + extra)
        getattr(lib, f"spion_{fam}_attn_forward").restype = None
        getattr(lib, f"spion_{fam}_attn_backward").argtypes = [_P] * 12
        getattr(lib, f"spion_{fam}_attn_backward").restype = None
        getattr(lib, f"spion_{fam}_destroy").argtypes = [_P]
        getattr(lib, f"spion_{fam}_destroy").restype = None
    lib._spion_typed = True
    return lib


def transpose_last2(x):
    """[..., R, C] fp32 CUDA tensor -> new contiguous [..., C, R] tensor (the library's tiled transpose)."""
    x = x.contiguous()
    R, C = x.shape[-2], x.shape[-1]
    batch = x.numel() // (R * C) if x.numel() else 0
    out = torch.empty(x.shape[:-2] + (C, R), dtype=torch.float32, device=x.device)
    if batch == 0:
        return out
    if batch > 65535:
        return x.transpose(-1, -2).contiguous()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    if core().spion_transpose_last2(x.data_ptr(), out.data_ptr(), batch, R, C, stream) != 0:
        check_error("spion_transpose_last2")
    return out


class HeadLayout(ctypes.Structure):
    """``spion_head_layout``: where element (b, h, i, f) of a [B, H, L, d] view lies, in floats."""

    _fields_ = [("batch_stride", ctypes.c_longlong), ("head_stride", c_int), ("row_stride", c_int)]


def head_layout(t: "torch.Tensor") -> HeadLayout | None:
    """Layout of a 4-D [B, H, L, d] tensor or view for the strided entry points; None when they cannot take it
    (last dimension not unit-stride, strides not multiples of 16 bytes, storage offset not 16-byte aligned)."""
    sb, sh, sl, sf = t.stride()
    if t.dim() != 4 or sf != 1 or t.data_ptr() % 16:
        return None
    unit = 16 // t.element_size()  # strides in elements, 16-byte granularity: 4 floats, 8 bf16
    if sb % unit or sh % unit or sl % unit or sl < t.shape[3] or min(sb, sh) < 0:
        return None
    if t.shape[2] * sl >= 1 << 29:
        return None
    return HeadLayout(sb, sh, sl)


def adjacent_head_views(q, k, v):
    """True when q, k, v ([B,H,L,d] views) are the three slices of one [B, L, 3, H, d] buffer, in this order."""
    B, H, L, d = q.shape
    strides = (L * 3 * H * d, d, 3 * H * d, 1)
    step = H * d * q.element_size()
    return (q.stride() == strides and k.stride() == strides and v.stride() == strides
            and k.data_ptr() - q.data_ptr() == step and v.data_ptr() - k.data_ptr() == step)


def empty_adjacent_heads(B, H, L, d, device):
    """Three uninitialised [B,H,L,d] views that are the slices of one [B, L, 3, H, d] buffer."""
    buf = torch.empty((B, L, 3, H, d), dtype=torch.float32, device=device)
    return tuple(buf[:, :, i].transpose(1, 2) for i in range(3))


def use_current_stream(module, device) -> None:
    """Point the module's handle at torch's current stream on ``device`` (the reference runs on the legacy
    default stream only): what makes the modules usable on side streams and under HIP graph capture.  One
    ctypes call per forward / backward; not cached, since handles can be shared or their addresses reused.
    (The raw-stream query is the one torch's own compiled code uses; ``torch.cuda.current_stream`` builds a Python
    stream object per call, 15 us on a slow host.)"""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    core().spion_set_stream(module.attn_handle, _raw_stream(index))


def _raw_stream_fallback(index: int) -> int:
    return torch.cuda.current_stream(index).cuda_stream


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", _raw_stream_fallback)


def check_error(where: str = "") -> None:
    """Raise if the library recorded a failure since the last check (the C entry points return void)."""
    lib = core()
    if not lib.spion_error_pending():
        return
    text = lib.spion_last_error().decode("utf-8", "replace")
    lib.spion_clear_error()
    raise SpionLibraryError(f"{where}: {text}" if where else text)


def load_dropin(name: str, n_init: int, n_fwd: int, n_bwd: int, trailing_int: bool) -> ctypes.CDLL:
    """Load one drop-in library and declare the ABI exactly as the reference's loaders do
    (models/attention.py:141-191): ``init`` takes ``n_init`` ints and returns an opaque pointer,
    ``attn_forward`` / ``attn_backward`` take ``n_fwd`` / ``n_bwd`` pointers (plus ``nnz`` for the
    block libraries), ``destroy`` takes the handle."""
    core()  # the drop-ins depend on libspion_hip.so; load it (and fail) first
    lib = _cdll(name)
    if getattr(lib, "_spion_typed", False):
        return lib
    tail = [c_int] if trailing_int else []
    lib.init.argtypes = [c_int] * n_init
    lib.init.restype = _P
    lib.attn_forward.argtypes = [_P] * n_fwd + tail
    lib.attn_forward.restype = None
    lib.attn_backward.argtypes = [_P] * n_bwd + tail
    lib.attn_backward.restype = None
    lib.destroy.argtypes = [_P]
    lib.destroy.restype = None
    lib._spion_typed = True
    return lib
