"""CPU-only checks of the C ABI library and the host logic (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mustafar_amd", "libmustafar_hip.so")
HEADER = os.path.join(ROOT, "include", "mustafar_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mstf_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        from mustafar_amd import build
        build.build()
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for must in ("mstf_prune_rows_f16", "mstf_compress_key_f16", "mstf_compress_value_f16", "mstf_key_spmv_f16",
                 "mstf_value_spmv_f16", "mstf_scale_softmax_f16", "mstf_compress_key_quant", "mstf_compress_value_quant",
                 "mstf_key_spmv_quant", "mstf_value_spmv_quant", "mstf_strerror"):
        assert must in syms


def test_library_exports_every_declared_symbol(lib):
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_binding_table_matches_header():
    from mustafar_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_error_strings_and_version(lib):
    lib.mstf_strerror.restype = ctypes.c_char_p
    assert lib.mstf_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert lib.mstf_strerror(code) and lib.mstf_strerror(code) != lib.mstf_strerror(-99)
    assert lib.mstf_version() >= 100


def test_argument_validation_returns_before_any_launch(lib):
    """Null pointers / bad shapes are rejected on the host; these calls never reach the GPU."""
    from mustafar_amd import _lib
    L = _lib.lib()
    assert L.mstf_key_spmv_f16(None, None, None, None, None, None, None, 64, 128, 1, 1, 1) == -1
    assert L.mstf_value_spmv_f16(None, None, None, None, None, None, None, 128, 64, 1, 1, 1, None, 0) == -1
    assert L.mstf_prune_rows_f16(None, None, None, 64, 128, 10) == -1
    assert L.mstf_scale_softmax_f16(None, None, None, 1, 64, 64, 64, 128) == -1
    assert L.mstf_compress_key_f16(None, None, 1, 64, 128, 0, None, None, None, None, None, 0, None, 0) == -1
    assert L.mstf_compress_value_quant(None, None, 1, 64, 128, 0, 2, None, None, None, None, None, None, None, None, 0,
                                       None, 0) == -1
    src = _lib.ProjSource()                                   # all zero: no source pointer
    assert L.mstf_compress_proj_f16(None, None, 0, 64, 128, 89, None, None, None, None, None, 0, None, 0) == -1
    assert L.mstf_compress_proj_f16(None, ctypes.byref(src), 0, 64, 128, 89, None, None, None, None, None, 0, None, 0) == -1
    assert L.mstf_append_proj_f16(None, ctypes.byref(src), 1, 64, 128, 89, None, None, None, None, None, None, None, 0) == -1
    # a row stride whose 64-row span does not fit the loaders' 32-bit byte offsets is refused, not wrapped
    wide = _lib.ProjSource()
    wide.x, wide.batch, wide.heads, wide.rows = 256, 1, 1, 64
    wide.stride_batch, wide.stride_head, wide.stride_token = 0, 128, 1 << 25
    assert L.mstf_compress_proj_f16(None, ctypes.byref(wide), 1, 64, 128, 89, 256, 256, 256, 256, 256, 8192, 256, 1 << 20) == -3
    L.mstf_test_set_spin_limit(0)       # host-side state only
    L.mstf_test_set_spin_limit(-1)
    assert L.mstf_decode_attention_f16(None, *([None] * 11), 64, 128, 4, 4, None, 0) == -1
    # the entry point on the library's fixed scratch buffer refuses, on the host, what does not fit into it
    assert L.mstf_decode_attention_static_f16(None, *([256] * 10), None, 4096, 128, 1012, 4) == -6
    assert L.mstf_decode_attention_static_f16(None, *([None] * 11), 4096, 128, 256, 4) == -1
    assert L.mstf_decode_attention_splits(4096, 128, 256, 4) == 8
    assert L.mstf_decode_attention_splits(4096, 128, 1024, 4) == 2       # 16384 blocks: four per wavefront
    # workspace sizes are pure host arithmetic
    assert L.mstf_compress_workspace_bytes(64, 4096, 128) >= 64 * 64 * 4 + 64 * 4
    assert L.mstf_value_spmv_workspace_bytes(128, 4096, 256, 4, 1) % 256 == 0
    assert L.mstf_value_spmv_workspace_bytes(128, 100, 256, 4, 1) == 0          # tokens % 64
    assert L.mstf_compress_quant_workspace_bytes(0, 64, 128) == 0


def test_host_helpers():
    from mustafar_amd import ops
    assert [ops.kth_from_sparsity(s, 128) for s in (0.5, 0.7, 0.9, 0.0)] == [64, 89, 115, 1]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from mustafar_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_install_aliases_gives_the_reference_module_names():
    """The import lines of the reference's model files resolve to the mirrors, with the names their pybind modules
    export (kernel/kernel_wrapper/pybind.cpp:9-10, kernel_quant/kernel_wrapper/pybind_quant.cpp:10-176)."""
    import importlib
    import sys
    import mustafar_amd
    saved = {k: sys.modules.get(k) for k in ("mustafar_package", "mustafar_package_quant", "kernel", "kernel.compression",
                                             "kernel_quant", "kernel_quant.compression_quant")}
    try:
        mustafar_amd.install_aliases()
        mp = importlib.import_module("mustafar_package")
        mpq = importlib.import_module("mustafar_package_quant")
        compression = importlib.import_module("kernel.compression")
        compression_quant = importlib.import_module("kernel_quant.compression_quant")
        for name in ("mustafar_key_formulation", "mustafar_value_formulation"):
            assert callable(getattr(mp, name))
        for name in ("mustafar_key_formulation_quant", "mustafar_key_formulation_quant_meta",
                     "mustafar_value_formulation_quant", "mustafar_value_formulation_quant_decode_n1",
                     "mustafar_quant_sparse_forward", "mustafar_quant_sparse_forward_meta",
                     "mustafar_quant_sparse_value_forward", "mustafar_quant_sparse_value_forward_decode_n1"):
            assert callable(getattr(mpq, name))
        assert callable(compression.convert_key_batched) and callable(compression.convert_value_batched)
        assert callable(compression_quant.convert_key_batched_quant)
        assert callable(compression_quant.convert_value_batched_quant)
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
