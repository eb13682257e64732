"""The C-ABI library: it is built, loads, and exports exactly the entry points
include/xpu_graph_amd.h declares (no compute calls here: no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xpu_graph_amd.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xg_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for s in ("xg_rms_norm", "xg_layer_norm", "xg_add_rms_norm", "xg_add_layer_norm", "xg_slice_cat", "xg_addn",
              "xg_combo_sum", "xg_slice_sum_cat", "xg_silu_mul", "xg_silu_mul2", "xg_dense", "xg_dense_glu", "xg_dense_fp8", "xg_sdpa", "xg_rope", "xg_copy_bytes",
              "xg_version", "xg_status_string"):
        assert s in syms


def test_library_exports_every_declared_symbol():
    from xpu_graph_amd import _lib

    if not _lib.is_built():
        pytest.fail(f"{_lib.LIB_PATH} not built: run `python -m xpu_graph_amd.build`")
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.exported_symbols()) == declared_symbols()  # the ctypes table covers the whole header


def test_status_strings_and_version():
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    assert lib.xg_version() >= 100
    assert lib.xg_status_string(0) == b"ok"
    assert b"NULL" in lib.xg_status_string(-4)
    with pytest.raises(_lib.XgError):
        _lib.check(-2, "demo")


def test_argument_validation_needs_no_gpu():
    """Host-side checks run before any launch, so they can be exercised without a device."""
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    assert lib.xg_rms_norm(None, None, None, 4, 8, 8, 1e-6, 0, 0, None) == -4  # NULL x
    buf = ctypes.create_string_buffer(1024)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.xg_rms_norm(p, None, p, 4, 8, 4, 1e-6, 0, 0, None) == -2  # stride < cols
    assert lib.xg_rms_norm(p, None, p, 4, 8, 8, 1e-6, 7, 7, None) == -1  # unknown dtype
    assert lib.xg_rms_norm(p, None, p, 0, 8, 8, 1e-6, 0, 0, None) == 0  # empty: nothing to launch
    assert lib.xg_copy_bytes(p, p, 24, None) == -2  # not a multiple of 16
    i32 = ctypes.c_int32 * 3
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, None, None, 3, 0, None) == -4  # NULL bounds
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 4, i32(0, 0, 0), i32(1, 2, 3), 3, 0, None) == -2  # row stride < cols
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 5), 3, 0, None) == -2  # end past the rows
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 3), 3, 9, None) == -1  # unknown dtype
    assert lib.xg_slice_sum_cat(p, p, 0, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 3), 3, 0, None) == 0  # empty batch
    assert lib.xg_silu_mul(p, p, 2, 8, 8, 0, None) == -2  # row stride < 2*d


def test_a_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    from xpu_graph_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libxpu_graph_amd.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.lib()


def test_the_ops_have_no_cpu_kernel():
    import torch

    import xpu_graph_amd.ops  # noqa: F401  registers torch.ops.xpu_ops.*

    x = torch.randn(4, 8)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.xpu_ops.rms_norm(x, torch.ones(8), 1e-6)
