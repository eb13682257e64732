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
    for s in ("xg_rms_norm", "xg_layer_norm", "xg_add_rms_norm", "xg_add_layer_norm", "xg_rms_norm_bwd", "xg_layer_norm_bwd", "xg_slice_cat", "xg_addn",
              "xg_combo_sum", "xg_slice_sum_cat", "xg_silu_mul", "xg_silu_mul2", "xg_silu_mul2_bwd", "xg_activation", "xg_activation_bwd", "xg_dense", "xg_dense_batched", "xg_dense_at", "xg_dense_glu", "xg_dense_glu_save", "xg_dense_fp8", "xg_slice_cat_check_table", "xg_sdpa", "xg_sdpa_masked", "xg_sdpa_lse", "xg_sdpa_backward", "xg_sdpa_masked_lse", "xg_sdpa_backward_masked", "xg_sdpa_decode", "xg_sdpa_decode_workspace_floats", "xg_sdpa_backward_static", "xg_rope", "xg_copy_bytes", "xg_clock_probe", "xg_wall_clock_khz",
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
    assert lib.xg_clock_probe(None, 4, 2000, None) == -4  # NULL output
    assert lib.xg_clock_probe(p, 4, 0, None) == -7  # empty window
    assert lib.xg_clock_probe(p, 1 << 20, 2000, None) == -7  # more windows than the probe takes
    assert lib.xg_clock_probe(p, 0, 2000, None) == 0  # nothing to launch
    i32 = ctypes.c_int32 * 3
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, None, None, 3, 0, None) == -4  # NULL bounds
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 4, i32(0, 0, 0), i32(1, 2, 3), 3, 0, None) == -2  # row stride < cols
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 5), 3, 0, None) == -2  # end past the rows
    assert lib.xg_slice_sum_cat(p, p, 2, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 3), 3, 9, None) == -1  # unknown dtype
    assert lib.xg_slice_sum_cat(p, p, 0, 4, 8, 32, 8, i32(0, 0, 0), i32(1, 2, 3), 3, 0, None) == 0  # empty batch
    assert lib.xg_silu_mul(p, p, 2, 8, 8, 0, None) == -2  # row stride < 2*d


def test_slice_table_is_refused_on_the_host_without_a_launch():
    """xg_slice_cat cannot look at its device-side table; xg_slice_cat_check_table refuses a bad HOST copy when the
    table is built: offsets outside the source row / the output row, an unknown output, a misaligned entry."""
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    i64 = ctypes.c_int64

    def check(entries, chunk=16, src_valid=256, out_valid=(64,)):
        arr = (_lib.XgChunk * len(entries))(*[_lib.XgChunk(*e, 0) for e in entries])
        valid = (i64 * len(out_valid))(*out_valid)
        return lib.xg_slice_cat_check_table(ctypes.cast(arr, ctypes.c_void_p), len(entries), chunk, src_valid, valid, len(out_valid))

    assert check([(0, 0, 0), (240, 48, 0)]) == 0
    assert check([(244, 0, 0)]) == -2  # reads past the source row
    assert check([(0, 52, 0)]) == -2  # writes past the output row
    assert check([(0, 0, 1)]) == -2  # no such output
    assert check([(-4, 0, 0)]) == -2
    assert check([(2, 0, 0)]) == -3  # source offsets need 4-byte alignment for 16-byte chunks
    assert check([(0, 8, 0)]) == -3  # output offsets are whole chunks
    assert check([(0, 0, 0)], chunk=3) == -7
    assert check([], chunk=16) == 0
    assert lib.xg_slice_cat_check_table(None, 1, 16, 256, (i64 * 1)(64), 1) == -4


def test_build_slice_table_runs_the_host_check():
    import torch  # noqa: F401

    from xpu_graph_amd import ops

    table, chunk, out_cols = ops.build_slice_table([[(3, 35), (100, 132)]], 8192, 4, 8192)
    assert chunk == 16 and out_cols == [64] and table.shape == (16, 4)
    with pytest.raises(ValueError):
        ops.build_slice_table([[(8190, 8200)]], 8192, 4, 8192)


def test_batched_dense_validation_needs_no_gpu():
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    buf = ctypes.create_string_buffer(1 << 16)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    ok = dict(batch=2, M=16, N=16, K=16, lda=16, ldb=16, ldr=0, sa=256, sb=256, sbias=0, sres=0, sout=256)

    def call(**kw):
        a = {**ok, **kw}
        return lib.xg_dense_batched(p, p, None, None, p, a["batch"], a["M"], a["N"], a["K"], a["lda"], a["ldb"], a["ldr"], a["sa"], a["sb"],
                                    a["sbias"], a["sres"], a["sout"], 0, 0, 2, 2, None)

    assert call(batch=0) == 0  # nothing to launch
    assert call(M=0) == 0
    assert call(batch=-1) == -2
    assert call(sout=255) == -2  # entries of the output would overlap
    assert call(sa=260) == -3  # an entry would start off a 16-byte boundary
    assert call(batch=70000) == -5
    assert call(K=12) == -3
    assert lib.xg_dense_batched(None, p, None, None, p, 2, 16, 16, 16, 16, 16, 0, 256, 256, 0, 0, 256, 0, 0, 2, 2, None) == -4


def test_transposed_left_operand_validation_needs_no_gpu():
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    buf = ctypes.create_string_buffer(1 << 12)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    ok = dict(M=16, N=16, K=5, lda=16, ldb=16, ldr=0, dtype=2)

    def call(**kw):
        a = {**ok, **kw}
        return lib.xg_dense_at(p, p, None, p, a["M"], a["N"], a["K"], a["lda"], a["ldb"], a["ldr"], a["dtype"], None)

    assert call(M=12) == -3  # 16-byte loads along M
    assert call(N=20, ldb=24) == -3
    assert call(lda=8) == -2  # rows narrower than M
    assert call(K=0) == -2
    assert call(dtype=0) == -1  # fp32 has no kernel
    assert lib.xg_dense_at(None, p, None, p, 16, 16, 8, 16, 16, 0, 2, None) == -4
    off = ctypes.c_void_p(p.value + 2)
    assert lib.xg_dense_at(off, p, None, p, 16, 16, 8, 16, 16, 0, 2, None) == -3


def test_static_workspace_backward_refuses_more_rows_than_it_holds_without_a_gpu():
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    S3 = ctypes.c_int64 * 3
    p = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    args = (S3(), S3(), S3(), S3(), S3(), S3(), S3(), S3(), 1.0, 0, 2, None)
    assert lib.xg_sdpa_backward_static(p, p, p, p, p, p, p, p, p, 1, 1, 1, (1 << 21) + 1, 64, 64, *args) == -5
    assert lib.xg_sdpa_backward_static(p, p, p, p, p, p, p, p, p, 1 << 11, 1 << 11, 1, 1, 64, 64, *args) == -5
    assert lib.xg_sdpa_backward_static(p, p, p, p, p, p, p, p, p, 0, 4, 4, 64, 64, 64, *args) == 0  # nothing to do


def test_masked_backward_validation_needs_no_gpu():
    """The mask operand of the backward call is checked like the forward's: strides present, dtype fp32 or the
    tensors', rows that do not overlap; the device scale must be 4-byte aligned.  No pointer is dereferenced."""
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    S3 = ctypes.c_int64 * 3
    p = ctypes.c_void_p(256)
    st = S3(64 * 64 * 4, 64 * 64, 64)
    shape = (1, 4, 4, 64, 64, 64, st, st, st, st, st, st, st, st, 0.125, 0, 2, None)

    def call(mask, mask_strides, mask_dtype, scale_dev):
        return lib.xg_sdpa_backward_masked(p, p, p, p, p, p, mask, mask_strides, mask_dtype, scale_dev, p, p, p, p, *shape)

    assert call(p, None, 2, None) == -4              # a mask without strides
    assert call(p, S3(0, 0, 64), 1, None) == -1      # bf16 tensors, an fp16 mask (neither bf16 nor fp32)
    assert call(p, S3(0, 0, 32), 2, None) == -2      # mask rows of 64 keys at a pitch of 32 overlap
    assert call(p, S3(0, 0, -64), 2, None) == -2
    assert call(ctypes.c_void_p(257), S3(0, 0, 64), 2, None) == -3
    assert call(None, None, 2, ctypes.c_void_p(258)) == -3
    assert lib.xg_sdpa_masked_lse(p, p, p, p, None, None, None, 2, None, 1, 4, 4, 64, 64, 64, st, st, st, st, 0.125, 0, 2, None) == -4


def test_decode_attention_validation_and_workspace_size_need_no_gpu():
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    S3 = ctypes.c_int64 * 3
    p = ctypes.c_void_p(256)
    st = S3(32 * 4096 * 128, 4096 * 128, 128)
    tail = (st, st, st, st, 0.1, 2, None)

    def call(B, H, Hkv, Sq, Skv, D, v=p, mask=None, mask_strides=None, mask_dtype=2, scale_dev=None, ws=None, ws_floats=0, tail=tail):
        return lib.xg_sdpa_decode(p, p, v, p, None, mask, mask_strides, mask_dtype, scale_dev, ws, ws_floats, B, H, Hkv, Sq, Skv, D, *tail)

    assert call(1, 32, 32, 33, 4096, 128) == -2   # more rows than a workgroup holds
    assert call(1, 32, 32, 1, 4096, 96) == -2     # head size
    assert call(1, 32, 5, 1, 4096, 128) == -2     # heads do not divide
    assert call(1, 32, 32, 1, 4096, 128, v=None) == -4
    assert call(1, 32, 32, 1, 4096, 128, tail=(st, st, st, st, 0.1, 0, None)) == -1  # fp32 tensors
    assert call(1, 32, 32, 1, 4096, 128, ws=ctypes.c_void_p(260), ws_floats=1 << 20) == -3
    assert call(1, 32, 32, 1, 4096, 128, mask=p) == -4                                 # a mask without strides
    assert call(1, 32, 32, 1, 4096, 128, mask=p, mask_strides=S3(0, 0, 0), mask_dtype=1) == -1
    assert call(1, 32, 32, 2, 4096, 128, mask=p, mask_strides=S3(0, 0, 100)) == -2     # mask rows overlap
    assert call(1, 32, 32, 1, 4096, 128, scale_dev=ctypes.c_void_p(258)) == -3
    assert call(0, 32, 32, 1, 4096, 128) == 0     # nothing to do
    # 32 problems of 32 tiles on 256 compute units: 8 key ranges of four tiles each, 32 x 128 + 64 floats per range
    assert lib.xg_sdpa_decode_workspace_floats(1, 32, 32, 1, 4096, 128) == 32 * 8 * (32 * 128 + 64)
    assert lib.xg_sdpa_decode_workspace_floats(64, 32, 32, 1, 4096, 128) == 0                     # 2048 problems fill the chip as they are
    assert lib.xg_sdpa_decode_workspace_floats(1, 32, 32, 33, 4096, 128) == 0


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
