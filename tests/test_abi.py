"""The built libraries load and export the declared C ABI; host-side argument checks (no GPU needed)."""
import ctypes
import os
import re

import pytest

from spion_amd import _lib
from spion_amd.attention import Attention

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    inc = os.path.join(ROOT, "include")
    headers = sorted(f for f in os.listdir(inc) if f.endswith(".h"))
    assert "spion_hip.h" in headers
    lib = ctypes.CDLL(_lib.lib_path("libspion_hip.so"))
    total = 0
    for h in headers:
        names = sorted(set(re.findall(r"\b(spion_\w+)\s*\(", open(os.path.join(inc, h)).read())))
        total += len(names)
        for n in names:
            assert hasattr(lib, n), f"{n} declared in include/{h} but not exported"
    assert total >= 30


@pytest.mark.parametrize("loader", ["_cuda_compile_module", "_cuda_mask_compile_module",
                                    "_blockcuda_compile_module", "_blockcuda_mask_compile_module"])
def test_dropins_export_reference_names(loader):
    lib = getattr(Attention, loader)()
    for n in ("init", "attn_forward", "attn_backward", "destroy"):
        assert hasattr(lib, n)


def test_init_validation_and_error_slot():
    core = _lib.core()
    core.spion_clear_error()
    assert core.spion_last_error() == b""
    assert not core.spion_block_init(0, 128, 4, 32)
    assert b"positive" in core.spion_last_error()
    core.spion_clear_error()
    assert not core.spion_block_init(33, 128, 4, 32)
    with pytest.raises(_lib.SpionLibraryError, match="emb_dim"):
        _lib.check_error("init")
    assert core.spion_last_error() == b""
    assert not core.spion_dense_init(32, 100, 4)      # L not a multiple of 32
    with pytest.raises(_lib.SpionLibraryError):
        _lib.check_error()
    h = core.spion_block_init(32, 128, 4, 32)
    assert h
    assert core.spion_last_path(h) == 0
    # a sparse handle handed to a dense entry point is rejected, nothing is launched
    core.spion_dense_attn_forward(h, None, None, None, None, None)
    with pytest.raises(_lib.SpionLibraryError, match="not a dense"):
        _lib.check_error()
    # null pointers are rejected before any GPU work
    core.spion_block_attn_forward(h, None, None, None, None, None, None, None, None, 0)
    with pytest.raises(_lib.SpionLibraryError, match="null pointer"):
        _lib.check_error()
    core.spion_block_destroy(h)
    core.spion_block_attn_forward(None, None, None, None, None, None, None, None, None, 0)
    with pytest.raises(_lib.SpionLibraryError, match="handle"):
        _lib.check_error()
    assert core.spion_pattern_generate(None, 1, 64, 32, 31, 0, 0.9, None, None, None, None) != 0
    with pytest.raises(_lib.SpionLibraryError, match="null"):
        _lib.check_error()
    assert core.spion_score_map_mean(None, 2, 2, 64, 1, None, None) != 0
    with pytest.raises(_lib.SpionLibraryError, match="spion_score_map_mean"):
        _lib.check_error()


def test_modules_refuse_to_run_without_library_handle():
    import spion_amd

    cfg = dict(head_dim=32, num_head=2, max_seq_len=128, batch_size=1, block_size=32)
    for cls in (spion_amd.CUDAAttention, spion_amd.CUDAMaskAttention, spion_amd.CUDABlockMaskAttention):
        with pytest.raises(_lib.SpionLibraryError):
            cls(cfg)
    with pytest.raises(_lib.SpionLibraryError):
        spion_amd.CUDABlockAttention(cfg, None, None)


def test_csr_builder_matches_oracle():
    import numpy as np
    from oracle import sparse_attention as osa
    from spion_amd.csr import block_mask_to_csr_host

    rng = np.random.default_rng(0)
    for nb, bs in ((4, 2), (7, 3), (8, 32), (5, 1)):
        mat = (rng.random((nb, nb)) < 0.4).astype(np.float32)
        mat[2, :] = 0
        a = block_mask_to_csr_host(mat, bs)
        b = osa.build_csr_from_block_mask(mat, bs)
        for x, y in zip(a, b):
            assert x.dtype == np.int32 and np.array_equal(x, y)


def test_autograd_node_library_loads_without_a_gpu():
    """lib/_spion_node.so (csrc/autograd_node.cpp, built by spion_amd.build against libtorch) imports and exposes
    the one function the modules call; no kernel is launched."""
    from spion_amd import _lib

    node = _lib.autograd_node()
    if node is None:
        pytest.skip("SPION_PY_NODE=1")
    assert callable(node.sparse_attention)
