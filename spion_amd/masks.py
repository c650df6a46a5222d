"""Block-mask persistence and the dense-to-sparse transition test of the training drivers.

* ``save_mask_list`` / ``load_mask_list``: the ``[4, layers, nb, nb]`` float32 tensor of block masks in the file
  format the reference writes and reads (a plain ``pickle.dump`` of the tensor, main_conv_ff.py:301-306,
  main_inference.py:164-166), so masks discovered by either side load into the other.  Loading goes through a
  restricted unpickler: only the handful of callables a pickled tensor needs are resolved, and the storage bytes
  are decoded with ``torch.load(..., weights_only=True)``; anything else in the file raises.
* ``TransitionDetector``: the test that ends the dense phase (main_conv_ff.py:211-242).  After every evaluation
  the head/batch-averaged score map of each layer is compared with the previous one; the Frobenius distance of
  consecutive maps is itself compared with the previous distance, and once it changed by less than 15 % (after
  truncation to an integer percentage) in every layer the pattern is considered settled.
"""
from __future__ import annotations

import io
import math
import pickle

import torch


def stack_for_replicas(layer_masks, replicas: int = 4) -> torch.Tensor:
    """[layers][nb, nb] masks -> [replicas, layers, nb, nb] (main_conv_ff.py:298-299: one copy per GPU replica)."""
    m = torch.stack([torch.as_tensor(x, dtype=torch.float32) for x in layer_masks], 0)
    return torch.stack([m] * replicas, 0)


def save_mask_list(mat_lst: torch.Tensor, path: str) -> None:
    if mat_lst.dim() != 4 or mat_lst.shape[-1] != mat_lst.shape[-2]:
        raise ValueError(f"expected [replicas, layers, nb, nb], got {tuple(mat_lst.shape)}")
    with open(path, "wb") as f:
        pickle.dump(mat_lst.detach().to(torch.float32).cpu().contiguous(), f, pickle.HIGHEST_PROTOCOL)


def _storage_from_bytes(b: bytes):
    # the reference pickles the tensor as it lies on the GPU (main_conv_ff.py:298-306): bring the bytes to the host,
    # whatever device tag they carry
    return torch.load(io.BytesIO(b), weights_only=True, map_location="cpu")


class _TensorOnlyUnpickler(pickle.Unpickler):
    _ALLOWED = {
        ("torch._utils", "_rebuild_tensor_v2"),
        ("torch._utils", "_rebuild_tensor"),
        ("collections", "OrderedDict"),
        ("torch", "FloatStorage"),
        ("torch", "device"),
    }

    def find_class(self, module, name):
        if (module, name) == ("torch.storage", "_load_from_bytes"):
            return _storage_from_bytes
        if (module, name) in self._ALLOWED:
            return super().find_class(module, name)
        raise pickle.UnpicklingError(f"mask file refers to {module}.{name}: not a plain float tensor")


def load_mask_list(path: str, device=None) -> torch.Tensor:
    with open(path, "rb") as f:
        obj = _TensorOnlyUnpickler(f).load()
    if not isinstance(obj, torch.Tensor) or obj.dim() != 4 or obj.shape[-1] != obj.shape[-2]:
        raise ValueError("mask file does not hold a [replicas, layers, nb, nb] tensor")
    obj = obj.to(torch.float32)
    return obj.to(device) if device is not None else obj


class TransitionDetector:
    """``update(attn_lst)`` after each evaluation; returns True from the call on which every layer's change of
    distance fell below ``percent`` (main_conv_ff.py:211-242).  ``attn_lst[l]`` is the layer's averaged score map."""

    def __init__(self, num_layers: int, percent: int = 15):
        self.num_layers = num_layers
        self.percent = percent
        self.before_attn: list = []
        self.before_distance: list = []
        self.diff: list = []
        self.transition = False

    def update(self, attn_lst) -> bool:
        if self.transition:
            return True
        cur = [attn_lst[l].detach() for l in range(self.num_layers)]
        if not self.before_attn:  # first evaluation: nothing to compare with
            self.before_attn = cur
            return False
        dist = [torch.sqrt(torch.sum(torch.pow(self.before_attn[l] - cur[l], 2))) for l in range(self.num_layers)]
        if not self.before_distance:  # second evaluation: first distance, no change yet; the reference map stays
            self.before_distance = dist
            self.diff = [0.0] * self.num_layers
            return False
        settled = 0
        for l in range(self.num_layers):
            self.diff[l] = float((abs(dist[l] - self.before_distance[l]) / self.before_distance[l]) * 100)
            self.before_distance[l] = dist[l]
            # a previous distance of 0 (two identical maps in a row) makes the change inf or NaN, on which the
            # reference's int(diff) raises: such a layer counts as not settled
            if math.isfinite(self.diff[l]) and int(self.diff[l]) < self.percent:
                settled += 1
        if settled == self.num_layers:
            self.transition = True
        else:
            self.before_attn = cur
        return self.transition


class DeviceTransitionDetector:
    """The same test with its state on the GPU (``spion_transition_update``): the distances, their comparison and
    the replacement of the kept maps run as three small kernels, and one float comes back per evaluation, where
    ``TransitionDetector`` synchronises on a reduction per layer.  ``update(attn_lst)`` takes the layers' averaged
    score maps ([L, L] CUDA tensors, or one stacked [layers, L, L] tensor) and returns the decision; ``diff`` and
    ``before_distance`` read the device state back for logging."""

    PARTIAL_BLOCKS = 256

    def __init__(self, num_layers: int, percent: int = 15):
        self.num_layers = num_layers
        self.percent = percent
        self.transition = False
        self._prev = None
        self._state = None
        self._partial = None

    def _state_host(self):
        return self._state.cpu().tolist() if self._state is not None else [0.0] * (2 * self.num_layers + 3)

    @property
    def before_distance(self):
        return self._state_host()[: self.num_layers]

    @property
    def diff(self):
        return self._state_host()[self.num_layers: 2 * self.num_layers]

    def update(self, attn_lst) -> bool:
        from . import _lib

        if self.transition:
            return True
        if isinstance(attn_lst, torch.Tensor):
            cur = attn_lst[: self.num_layers]
        else:
            cur = torch.stack([attn_lst[l].detach() for l in range(self.num_layers)], 0)
        cur = cur.detach().to(torch.float32).contiguous()
        if not cur.is_cuda:
            raise _lib.SpionLibraryError("DeviceTransitionDetector runs on the GPU only; got CPU tensors")
        if self._prev is None:
            self._prev = torch.empty_like(cur)
            self._state = torch.zeros(2 * self.num_layers + 3, dtype=torch.float32, device=cur.device)
            self._partial = torch.empty(self.num_layers * self.PARTIAL_BLOCKS, dtype=torch.float64, device=cur.device)
        elif self._prev.shape != cur.shape:
            raise ValueError(f"score maps changed shape: {tuple(self._prev.shape)} -> {tuple(cur.shape)}")
        stream = torch.cuda.current_stream(cur.device).cuda_stream
        rc = _lib.core().spion_transition_update(cur.data_ptr(), self._prev.data_ptr(), self.num_layers,
                                                 cur[0].numel(), self._state.data_ptr(), self._partial.data_ptr(),
                                                 self.PARTIAL_BLOCKS, self.percent, stream)
        if rc != 0:
            _lib.check_error("spion_transition_update")
        self.transition = bool(self._state[2 * self.num_layers + 1].item() != 0.0)  # the one read-back
        return self.transition
