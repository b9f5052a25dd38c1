"""The C-ABI library loads and exports every symbol include/llmk.h declares (no compute calls)."""
import ctypes
import os
import re

import pytest

from llm_kernels_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "llmk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llmk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), "missing export %s" % n


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == _declared()


def test_version_and_error_paths_without_gpu():
    lib = _lib.load()
    assert lib.llmk_version() >= 100
    # argument validation happens before any HIP call, so it is testable without a GPU
    rc = lib.llmk_gemm_fp8_block(None, None, None, None, None, 0, 16, 16, 100, None, 0, None)
    assert rc == -1 and b"multiple of 128" in lib.llmk_last_error()
    rc = lib.llmk_gemm_w4a16_marlin(None, None, None, None, 16, 48, 64, 16, None, 0, None)
    assert rc == -1 and b"multiple of 64" in lib.llmk_last_error()
    rc = lib.llmk_gemm_w4a16_marlin(None, None, None, None, 15, 64, 64, 16, None, 0, None)
    assert rc == -1
    # the entry point with the built-in scratch refuses shapes beyond it before touching the GPU
    rc = lib.llmk_gemm_fp8_block_static(256, 256, 256, 256, 256, 2, 16, 128256, 20480, None)
    assert rc == -1 and b"built-in" in lib.llmk_last_error()
    rc = lib.llmk_pack_rows(None, 1, None, 4, 4, 3, 32, None)
    assert rc == -2
    rc = lib.llmk_act_quant_i8(None, 0, None, None, 4, 100, 0, None)
    assert rc == -1


def test_product_refuses_cpu_tensors():
    import torch
    from llm_kernels_amd.quantization import fp8_kernel, bitpack
    with pytest.raises(_lib.LlmkError):
        fp8_kernel.act_quant(torch.randn(4, 128))
    with pytest.raises(_lib.LlmkError):
        bitpack.pack_weights_over_rows(torch.zeros(8, 8, dtype=torch.uint8), 4, 32, False)


def test_release_workspaces_drops_the_cached_scratch():
    saved = dict(_lib._ws)
    try:
        _lib._ws.clear()
        _lib._ws[(0, 11)] = object()
        _lib._ws[(0, 12)] = object()
        _lib._ws[(1, 11)] = object()
        _lib.release_workspaces("cuda:1")
        assert sorted(_lib._ws) == [(0, 11), (0, 12)]
        _lib.release_workspaces()
        assert not _lib._ws
    finally:
        _lib._ws.clear()
        _lib._ws.update(saved)
