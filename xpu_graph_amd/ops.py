"""``torch.ops.xpu_ops.*``: the custom ops the mi355x target modules call.

Each op has a schema, a Meta (fake-tensor) implementation so that the pass
pipeline can re-propagate shapes through rewritten graphs, and ONE real
implementation, registered for the CUDA dispatch key (HIP on ROCm), that hands
raw device pointers and the current stream to the C-ABI kernel library.  There
is deliberately no CPU implementation: calling an op on CPU tensors raises
NotImplementedError from the dispatcher.

Op names follow the reference's convention of a vendor op namespace allowed
inside device graphs (`xpu_ops`, src/xpu_graph/backends/device_graph.py:26-29).
"""
import ctypes
from typing import List, Optional

import torch

from . import _lib
from ._lib import XG_BF16, XG_F16, XG_F32

_DTYPE_CODE = {torch.float32: XG_F32, torch.float16: XG_F16, torch.bfloat16: XG_BF16}

_library = torch.library.Library("xpu_ops", "DEF")

_SCHEMAS = [
    "rms_norm(Tensor x, Tensor? weight, float eps) -> Tensor",
    "layer_norm(Tensor x, Tensor? weight, Tensor? bias, float eps) -> Tensor",
    "add_rms_norm(Tensor x, Tensor residual, Tensor? weight, float eps) -> (Tensor, Tensor)",
    "add_rms_norm_only(Tensor x, Tensor residual, Tensor? weight, float eps) -> Tensor",
    "add_layer_norm(Tensor x, Tensor residual, Tensor? weight, Tensor? bias, float eps) -> (Tensor, Tensor)",
    "add_layer_norm_only(Tensor x, Tensor residual, Tensor? weight, Tensor? bias, float eps) -> Tensor",
    "rms_norm_bwd(Tensor x, Tensor? residual, Tensor? weight, Tensor gy, Tensor? gh, float eps, bool want_gw) -> (Tensor, Tensor)",
    "layer_norm_bwd(Tensor x, Tensor? residual, Tensor? weight, Tensor gy, Tensor? gh, float eps, bool want_gw, bool want_gb) -> (Tensor, Tensor, Tensor)",
    "slice_cat(Tensor src, Tensor table, int chunk_bytes, int out_cols) -> Tensor",
    "slice_cat_multi(Tensor src, Tensor table, int chunk_bytes, int[] out_cols) -> Tensor[]",
    "slice_stack(Tensor src, Tensor[] tables, int[] chunk_bytes, int slice_len, int num) -> Tensor",
    "addn(Tensor[] inputs) -> Tensor",
    "combo_sum(Tensor[] inputs, int dim) -> Tensor[]",
    "slice_sum_cat(Tensor x, int[] starts, int[] ends) -> Tensor",
    "silu_mul(Tensor x) -> Tensor",
    "silu_mul2(Tensor gate, Tensor up) -> Tensor",
    "silu_mul2_bwd(Tensor gate, Tensor up, Tensor gy) -> (Tensor, Tensor)",
    "act(Tensor x, str act) -> Tensor",
    "act_bwd(Tensor z, Tensor gy, str act) -> Tensor",
]
for _s in _SCHEMAS:
    _library.define(_s)


def _stream():
    """The current stream of the current device as a raw handle.  The private accessors are what
    torch.cuda.current_stream() ends in; going through the Stream object costs about 4 us per call, a third of an
    op's host time."""
    return _raw_stream(_current_device())


try:
    _raw_stream = torch._C._cuda_getCurrentRawStream
    _current_device = torch._C._cuda_getDevice
except AttributeError:  # a torch build without these accessors

    def _raw_stream(index):
        return torch.cuda.current_stream(index).cuda_stream

    _current_device = torch.cuda.current_device


def _code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"xpu_ops: dtype {dtype} has no mi355x kernel") from None


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()  # ctypes turns the integer into the declared pointer type


def _rows_2d(x: torch.Tensor):
    """View x as [rows, cols] with unit column stride without copying when possible."""
    cols = x.shape[-1]
    if x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= cols:
        return x, x.shape[0], x.stride(0)
    xc = x if x.is_contiguous() else x.contiguous()
    rows = xc.numel() // cols if cols else 0
    return xc, rows, cols


def _param_dtype(x_dtype, *params):
    """Affine parameters are read either in the activation dtype or in fp32."""
    out = []
    want = None
    for p in params:
        if p is not None and p.dtype != x_dtype:
            want = torch.float32
    for p in params:
        if p is None:
            out.append(None)
            continue
        q = p
        if want is not None and q.dtype != want:
            q = q.to(want)
        out.append(q.contiguous())
    return out, (want or x_dtype)


# ------------------------------------------------------------------- norms
def _norm_impl(kind, x, residual, weight, bias, eps, want_h):
    (weight, bias), wb_dtype = _param_dtype(x.dtype, weight, bias)
    cols = x.shape[-1]
    for p in (weight, bias):
        if p is not None and p.numel() != cols:
            raise ValueError("xpu_ops norm: weight/bias must have the size of the last dimension")
    x2, rows, xs = _rows_2d(x)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    lib = _lib.lib()
    dt, wdt = _code(x.dtype), _code(wb_dtype)
    if x.numel() == 0:
        if residual is None or not want_h:
            return y
        return y, torch.empty_like(y)
    if residual is None:
        if kind == "rms":
            st = lib.xg_rms_norm(_ptr(x2), _ptr(weight), _ptr(y), rows, cols, xs, eps, dt, wdt, _stream())
        else:
            st = lib.xg_layer_norm(_ptr(x2), _ptr(weight), _ptr(bias), _ptr(y), rows, cols, xs, eps, dt, wdt, _stream())
        _lib.check(st, f"xg_{kind}_norm")
        return y
    if residual.shape != x.shape or residual.dtype != x.dtype:
        raise ValueError("xpu_ops add+norm: residual must match x in shape and dtype")
    r2, _, rs = _rows_2d(residual)
    h = torch.empty(x.shape, dtype=x.dtype, device=x.device) if want_h else None
    if kind == "rms":
        st = lib.xg_add_rms_norm(_ptr(x2), _ptr(r2), _ptr(weight), _ptr(y), _ptr(h), rows, cols, xs, rs, eps, dt, wdt, _stream())
    else:
        st = lib.xg_add_layer_norm(
            _ptr(x2), _ptr(r2), _ptr(weight), _ptr(bias), _ptr(y), _ptr(h), rows, cols, xs, rs, eps, dt, wdt, _stream()
        )
    _lib.check(st, f"xg_add_{kind}_norm")
    return (y, h) if want_h else y


def _rms_norm(x, weight, eps):
    return _norm_impl("rms", x, None, weight, None, eps, False)


def _layer_norm(x, weight, bias, eps):
    return _norm_impl("layer", x, None, weight, bias, eps, False)


def _add_rms_norm(x, residual, weight, eps):
    return _norm_impl("rms", x, residual, weight, None, eps, True)


def _add_rms_norm_only(x, residual, weight, eps):
    return _norm_impl("rms", x, residual, weight, None, eps, False)


def _add_layer_norm(x, residual, weight, bias, eps):
    return _norm_impl("layer", x, residual, weight, bias, eps, True)


def _add_layer_norm_only(x, residual, weight, bias, eps):
    return _norm_impl("layer", x, residual, weight, bias, eps, False)


_RMS_BWD_BLOCKS = 1024  # workgroups that split the rows; each hands back one fp32 partial row of the weight gradient


def rms_norm_bwd_fits(x, weight):
    """What xg_rms_norm_bwd takes: rows of whole 16-byte vectors, at most eight of them per lane of a 256-lane block,
    a weight that is one row."""
    per16 = 16 // x.element_size()
    cols = x.shape[-1]
    ok = x.dtype in _DTYPE_CODE and isinstance(cols, int) and cols % per16 == 0 and 0 < cols // per16 <= 2048
    if weight is not None:
        ok = ok and weight.dim() == 1 and weight.shape[0] == cols and weight.dtype in (x.dtype, torch.float32)
    return ok


def _rms_norm_bwd(x, residual, weight, gy, gh, eps, want_gw):
    """Gradients of rms_norm / add_rms_norm in one pass per row: (gx, gw); gx also is the residual's gradient.  gw is
    empty when there is no weight or want_gw is false."""
    if not rms_norm_bwd_fits(x, weight):
        raise ValueError("rms_norm_bwd: needs rows of whole 16-byte vectors (at most 2048 of them) and a 1-D weight")
    cols = x.shape[-1]
    x2, rows, xs = _rows_2d(x)
    g2, _, gs = _rows_2d(gy.to(x.dtype))
    r2 = rs = h2 = hs = None
    if residual is not None:
        r2, _, rs = _rows_2d(residual)
    if gh is not None:
        h2, _, hs = _rows_2d(gh.to(x.dtype))
    gx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    want_gw = bool(want_gw and weight is not None)
    n_blocks = max(1, min(_RMS_BWD_BLOCKS, rows))
    part = torch.empty((n_blocks, cols), dtype=torch.float32, device=x.device) if want_gw else None
    if rows:
        st = _lib.lib().xg_rms_norm_bwd(
            _ptr(x2), _ptr(r2), _ptr(weight.contiguous() if weight is not None else None), _ptr(g2), _ptr(h2), _ptr(gx), _ptr(part), rows, cols,
            xs, rs or 0, gs, hs or 0, eps, _code(x.dtype), _code(weight.dtype) if weight is not None else _code(x.dtype), n_blocks, _stream(),
        )
        _lib.check(st, "xg_rms_norm_bwd")
    if not want_gw:
        return gx, torch.empty(0, dtype=x.dtype, device=x.device)
    return gx, (part.sum(0) if rows else torch.zeros(cols, device=x.device)).to(weight.dtype)


def _layer_norm_bwd(x, residual, weight, gy, gh, eps, want_gw, want_gb):
    """Gradients of layer_norm / add_layer_norm in one pass per row: (gx, gw, gb); gx also is the residual's
    gradient.  gw / gb are empty when not wanted (or, for gw, when there is no weight); gb has the dtype of the
    weight when there is one, else that of x."""
    if not rms_norm_bwd_fits(x, weight):
        raise ValueError("layer_norm_bwd: needs rows of whole 16-byte vectors (at most 2048 of them) and a 1-D weight")
    cols = x.shape[-1]
    x2, rows, xs = _rows_2d(x)
    g2, _, gs = _rows_2d(gy.to(x.dtype))
    r2 = rs = h2 = hs = None
    if residual is not None:
        r2, _, rs = _rows_2d(residual)
    if gh is not None:
        h2, _, hs = _rows_2d(gh.to(x.dtype))
    gx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    want_gw = bool(want_gw and weight is not None)
    n_blocks = max(1, min(_RMS_BWD_BLOCKS, rows))
    # one buffer for both partial sums: its halves are summed by one reduction
    n_out = int(want_gw) + int(bool(want_gb))
    part = torch.empty((n_out, n_blocks, cols), dtype=torch.float32, device=x.device) if n_out else None
    pw = part[0] if want_gw else None
    pb = part[n_out - 1] if want_gb else None
    if rows:
        st = _lib.lib().xg_layer_norm_bwd(
            _ptr(x2), _ptr(r2), _ptr(weight.contiguous() if weight is not None else None), _ptr(g2), _ptr(h2), _ptr(gx), _ptr(pw), _ptr(pb),
            rows, cols, xs, rs or 0, gs, hs or 0, eps, _code(x.dtype), _code(weight.dtype) if weight is not None else _code(x.dtype), n_blocks,
            _stream(),
        )
        _lib.check(st, "xg_layer_norm_bwd")
    wdt = weight.dtype if weight is not None else x.dtype
    none = torch.empty(0, dtype=x.dtype, device=x.device)
    if not n_out:
        return gx, none, none
    sums = part.sum(1) if rows else torch.zeros((n_out, cols), device=x.device)
    return gx, (sums[0].to(wdt) if want_gw else none), (sums[n_out - 1].to(wdt) if want_gb else none)


def _layer_norm_bwd_meta(x, residual, weight, gy, gh, eps, want_gw, want_gb):
    gx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    wdt = weight.dtype if weight is not None else x.dtype
    none = torch.empty(0, dtype=x.dtype, device=x.device)
    row = lambda: torch.empty((x.shape[-1],), dtype=wdt, device=x.device)  # noqa: E731
    return gx, (row() if want_gw and weight is not None else none), (row() if want_gb else none)


def _rms_norm_bwd_meta(x, residual, weight, gy, gh, eps, want_gw):
    gx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if want_gw and weight is not None:
        return gx, torch.empty(weight.shape, dtype=weight.dtype, device=x.device)
    return gx, torch.empty(0, dtype=x.dtype, device=x.device)


def _like(x):
    return torch.empty(x.shape, dtype=x.dtype, device=x.device)


_library.impl("rms_norm", _rms_norm, "CUDA")
_library.impl("layer_norm", _layer_norm, "CUDA")
_library.impl("rms_norm_bwd", _rms_norm_bwd, "CUDA")
_library.impl("rms_norm_bwd", _rms_norm_bwd_meta, "Meta")
_library.impl("layer_norm_bwd", _layer_norm_bwd, "CUDA")
_library.impl("layer_norm_bwd", _layer_norm_bwd_meta, "Meta")
_library.impl("add_rms_norm", _add_rms_norm, "CUDA")
_library.impl("add_rms_norm_only", _add_rms_norm_only, "CUDA")
_library.impl("add_layer_norm", _add_layer_norm, "CUDA")
_library.impl("add_layer_norm_only", _add_layer_norm_only, "CUDA")
_library.impl("rms_norm", lambda x, weight, eps: _like(x), "Meta")
_library.impl("layer_norm", lambda x, weight, bias, eps: _like(x), "Meta")
_library.impl("add_rms_norm", lambda x, residual, weight, eps: (_like(x), _like(x)), "Meta")
_library.impl("add_rms_norm_only", lambda x, residual, weight, eps: _like(x), "Meta")
_library.impl("add_layer_norm", lambda x, residual, weight, bias, eps: (_like(x), _like(x)), "Meta")
_library.impl("add_layer_norm_only", lambda x, residual, weight, bias, eps: _like(x), "Meta")


# --------------------------------------------------------------- slice / cat
def _slice_cat_multi(src, table, chunk_bytes, out_cols):
    if src.dim() != 2:
        raise NotImplementedError("input must be 2d")
    if src.stride(1) != 1:
        src = src.contiguous()
    esz = src.element_size()
    rows = src.shape[0]
    outs = [torch.empty((rows, c), dtype=src.dtype, device=src.device) for c in out_cols]
    n = len(outs)
    if n > _lib.SLICE_CAT_MAX_OUTS:
        raise ValueError(f"slice_cat_multi: at most {_lib.SLICE_CAT_MAX_OUTS} outputs per call")
    if table.dtype != torch.int32 or table.dim() != 2 or table.shape[1] != 4 or not table.is_contiguous():
        raise ValueError("slice_cat: table must be a contiguous int32 [n_chunks, 4] tensor")
    if table.device != src.device:
        raise ValueError("slice_cat: table must live on the source's device")
    if rows == 0 or table.shape[0] == 0:
        return outs
    align = min(chunk_bytes, 4)
    if (src.stride(0) * esz) % align or src.data_ptr() % align:
        src = src.contiguous()
    ptrs = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    rbs = (ctypes.c_int64 * n)(*[c * esz for c in out_cols])
    st = _lib.lib().xg_slice_cat(
        _ptr(src), src.stride(0) * esz, rows, ptrs, rbs, n, _ptr(table), table.shape[0], chunk_bytes, _stream()
    )
    _lib.check(st, "xg_slice_cat")
    return outs


def _slice_cat(src, table, chunk_bytes, out_cols):
    return _slice_cat_multi(src, table, chunk_bytes, [out_cols])[0]


def _slice_stack(src, tables, chunk_bytes, slice_len, num):
    """[num, rows, slice_len]: slab k holds one column slice of `src`.  tables[g] places the slices
    [g * MAX_OUTS, (g + 1) * MAX_OUTS) as the outputs of one `xg_slice_cat` launch; every output pointer is a slab
    of the ONE result buffer."""
    if src.dim() != 2:
        raise NotImplementedError("input must be 2d")
    if src.stride(1) != 1:
        src = src.contiguous()
    esz = src.element_size()
    rows = src.shape[0]
    out = torch.empty((num, rows, slice_len), dtype=src.dtype, device=src.device)
    step = _lib.SLICE_CAT_MAX_OUTS
    if len(tables) != (num + step - 1) // step or len(chunk_bytes) != len(tables):
        raise ValueError("slice_stack: one table and one chunk size per group of outputs")
    if out.numel() == 0:
        return out
    align = min(min(chunk_bytes), 4)
    if (src.stride(0) * esz) % align or src.data_ptr() % align:
        src = src.contiguous()
    slab = rows * slice_len * esz
    for g, (table, chunk) in enumerate(zip(tables, chunk_bytes)):
        n = min(step, num - g * step)
        if table.dtype != torch.int32 or table.dim() != 2 or table.shape[1] != 4 or not table.is_contiguous():
            raise ValueError("slice_stack: tables must be contiguous int32 [n_chunks, 4] tensors")
        if table.device != src.device:
            raise ValueError("slice_stack: tables must live on the source's device")
        ptrs = (ctypes.c_void_p * n)(*[out.data_ptr() + (g * step + k) * slab for k in range(n)])
        rbs = (ctypes.c_int64 * n)(*([slice_len * esz] * n))
        st = _lib.lib().xg_slice_cat(_ptr(src), src.stride(0) * esz, rows, ptrs, rbs, n, _ptr(table), table.shape[0], chunk, _stream())
        _lib.check(st, "xg_slice_cat")
    return out


_library.impl("slice_cat", _slice_cat, "CUDA")
_library.impl("slice_stack", _slice_stack, "CUDA")
_library.impl(
    "slice_stack",
    lambda src, tables, chunk_bytes, slice_len, num: torch.empty((num, src.shape[0], slice_len), dtype=src.dtype, device=src.device),
    "Meta",
)
_library.impl("slice_cat_multi", _slice_cat_multi, "CUDA")
_library.impl(
    "slice_cat",
    lambda src, table, chunk_bytes, out_cols: torch.empty((src.shape[0], out_cols), dtype=src.dtype, device=src.device),
    "Meta",
)
_library.impl(
    "slice_cat_multi",
    lambda src, table, chunk_bytes, out_cols: [
        torch.empty((src.shape[0], c), dtype=src.dtype, device=src.device) for c in out_cols
    ],
    "Meta",
)


# --------------------------------------------------------------------- sums
def _addn(inputs: List[torch.Tensor]):
    if len(inputs) == 0:
        raise ValueError("addn: needs at least one input")
    first = inputs[0]
    ins = []
    for t in inputs:
        if t.shape != first.shape or t.dtype != first.dtype:
            raise ValueError("addn: all inputs must share shape and dtype")
        ins.append(t if t.is_contiguous() else t.contiguous())
    out = torch.empty(first.shape, dtype=first.dtype, device=first.device)
    if out.numel() == 0:
        return out
    ptrs = (ctypes.c_void_p * len(ins))(*[t.data_ptr() for t in ins])
    st = _lib.lib().xg_addn(ptrs, len(ins), _ptr(out), out.numel(), _code(first.dtype), _stream())
    _lib.check(st, "xg_addn")
    return out


def _combo_sum_shapes(inputs, dim):
    if dim not in (1, 2):
        raise ValueError("combo_sum: dim must be 1 or 2")
    shapes = []
    for t in inputs:
        if t.dim() != 3:
            raise ValueError("combo_sum: inputs must be 3-d")
        shapes.append((t.shape[0], t.shape[2]) if dim == 1 else (t.shape[0], t.shape[1]))
    return shapes


def _combo_sum(inputs: List[torch.Tensor], dim: int):
    shapes = _combo_sum_shapes(inputs, dim)
    if len(inputs) == 0:
        return []
    dtype = inputs[0].dtype
    ins = []
    for t in inputs:
        if t.dtype != dtype:
            raise ValueError("combo_sum: all inputs must share a dtype")
        ins.append(t if t.is_contiguous() else t.contiguous())
    outs = [torch.empty(s, dtype=dtype, device=t.device) for s, t in zip(shapes, ins)]
    lib = _lib.lib()
    step = _lib.COMBO_SUM_MAX_JOBS
    for lo in range(0, len(ins), step):
        part_in, part_out = ins[lo : lo + step], outs[lo : lo + step]
        n = len(part_in)
        ip = (ctypes.c_void_p * n)(*[t.data_ptr() for t in part_in])
        op = (ctypes.c_void_p * n)(*[t.data_ptr() for t in part_out])
        s0 = (ctypes.c_int64 * n)(*[t.shape[0] for t in part_in])
        s1 = (ctypes.c_int64 * n)(*[t.shape[1] for t in part_in])
        s2 = (ctypes.c_int64 * n)(*[t.shape[2] for t in part_in])
        st = lib.xg_combo_sum(ip, op, s0, s1, s2, n, dim, _code(dtype), _stream())
        _lib.check(st, "xg_combo_sum")
    return outs


_library.impl("addn", _addn, "CUDA")
_library.impl("combo_sum", _combo_sum, "CUDA")


def _slice_sum_cat(x, starts, ends):
    """x [B, R, C] -> [B, n * C]; block i = x[:, starts[i]:ends[i], :].sum(1)."""
    if x.dim() != 3:
        raise NotImplementedError("input must be 3d")
    if len(starts) != len(ends) or len(starts) == 0:
        raise ValueError("slice_sum_cat: one (start, end) pair per slice, at least one")
    if len(starts) > _lib.SLICE_SUM_MAX_SLICES:
        raise ValueError(f"slice_sum_cat: at most {_lib.SLICE_SUM_MAX_SLICES} slices per call")
    if x.stride(2) != 1 or x.stride(1) < x.shape[2]:
        x = x.contiguous()
    B, R, C = x.shape
    n = len(starts)
    out = torch.empty((B, n * C), dtype=x.dtype, device=x.device)
    if out.numel() == 0:
        return out
    s_arr = (ctypes.c_int32 * n)(*starts)
    e_arr = (ctypes.c_int32 * n)(*ends)
    st = _lib.lib().xg_slice_sum_cat(_ptr(x), _ptr(out), B, R, C, x.stride(0), x.stride(1), s_arr, e_arr, n, _code(x.dtype), _stream())
    _lib.check(st, "xg_slice_sum_cat")
    return out


_library.impl("slice_sum_cat", _slice_sum_cat, "CUDA")
_library.impl(
    "slice_sum_cat",
    lambda x, starts, ends: torch.empty((x.shape[0], len(starts) * x.shape[2]), dtype=x.dtype, device=x.device),
    "Meta",
)
_library.impl("addn", lambda inputs: _like(inputs[0]), "Meta")
_library.impl(
    "combo_sum",
    lambda inputs, dim: [
        torch.empty(s, dtype=t.dtype, device=t.device) for s, t in zip(_combo_sum_shapes(inputs, dim), inputs)
    ],
    "Meta",
)


# ------------------------------------------------------------------- SwiGLU
def _silu_mul(x):
    if x.shape[-1] % 2 != 0:
        raise ValueError("silu_mul: last dimension must be even")
    d = x.shape[-1] // 2
    x2, rows, xs = _rows_2d(x)
    y = torch.empty((*x.shape[:-1], d), dtype=x.dtype, device=x.device)
    if y.numel() == 0:
        return y
    st = _lib.lib().xg_silu_mul(_ptr(x2), _ptr(y), rows, d, xs, _code(x.dtype), _stream())
    _lib.check(st, "xg_silu_mul")
    return y


def _silu_mul2(gate, up):
    if gate.shape != up.shape or gate.dtype != up.dtype:
        raise ValueError("silu_mul2: gate and up must match in shape and dtype")
    d = gate.shape[-1]
    g2, rows, gs = _rows_2d(gate)
    u2, _, us = _rows_2d(up)
    y = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    if y.numel() == 0:
        return y
    st = _lib.lib().xg_silu_mul2(_ptr(g2), _ptr(u2), _ptr(y), rows, d, gs, us, _code(gate.dtype), _stream())
    _lib.check(st, "xg_silu_mul2")
    return y


def _silu_mul2_bwd(gate, up, gy):
    """(d_gate, d_up) of silu(gate) * up for the upstream gradient gy, in one pass over the three tensors."""
    if gate.shape != up.shape or gate.shape != gy.shape or gate.dtype != up.dtype or gate.dtype != gy.dtype:
        raise ValueError("silu_mul2_bwd: gate, up and gy must match in shape and dtype")
    gate, up, gy = gate.contiguous(), up.contiguous(), gy.contiguous()
    d_gate, d_up = torch.empty_like(gate), torch.empty_like(gate)
    if gate.numel():
        st = _lib.lib().xg_silu_mul2_bwd(_ptr(gate), _ptr(up), _ptr(gy), _ptr(d_gate), _ptr(d_up), gate.numel(), _code(gate.dtype), _stream())
        _lib.check(st, "xg_silu_mul2_bwd")
    return d_gate, d_up


def _act_code(act):
    code = _lib.ACT_CODES.get(act)
    if not code:
        raise ValueError(f"act: unknown activation {act!r} (relu, gelu, silu, sigmoid)")
    return code


def _act(x, act):
    """An activation of the dense layer on its own (what the layer of a differentiated graph runs after its product)."""
    code = _act_code(act)
    x = x.contiguous()
    y = torch.empty_like(x)
    if x.numel():
        _lib.check(_lib.lib().xg_activation(_ptr(x), _ptr(y), x.numel(), code, _code(x.dtype), _stream()), "xg_activation")
    return y


def _act_bwd(z, gy, act):
    """gy * act'(z) in one pass."""
    code = _act_code(act)
    if z.shape != gy.shape or z.dtype != gy.dtype:
        raise ValueError("act_bwd: z and gy must match in shape and dtype")
    z, gy = z.contiguous(), gy.contiguous()
    gz = torch.empty_like(z)
    if z.numel():
        _lib.check(_lib.lib().xg_activation_bwd(_ptr(z), _ptr(gy), _ptr(gz), z.numel(), code, _code(z.dtype), _stream()), "xg_activation_bwd")
    return gz


_library.impl("act", _act, "CUDA")
_library.impl("act", lambda x, act: _like(x), "Meta")
_library.impl("act_bwd", _act_bwd, "CUDA")
_library.impl("act_bwd", lambda z, gy, act: _like(z), "Meta")
_library.impl("silu_mul", _silu_mul, "CUDA")
_library.impl("silu_mul2", _silu_mul2, "CUDA")
_library.impl("silu_mul2_bwd", _silu_mul2_bwd, "CUDA")
_library.impl("silu_mul2_bwd", lambda gate, up, gy: (_like(gate), _like(gate)), "Meta")
_library.impl(
    "silu_mul",
    lambda x: torch.empty((*x.shape[:-1], x.shape[-1] // 2), dtype=x.dtype, device=x.device),
    "Meta",
)
_library.impl("silu_mul2", lambda gate, up: _like(gate), "Meta")


# ------------------------------------------------------------ slice tables
def build_slice_table(slice_lists, src_cols, elem_size, src_row_stride=None):
    """Chunk table for `xg_slice_cat` from static python slice lists.

    slice_lists: one list of (start, end) column ranges per output (already
    normalised to 0 <= start <= end <= src_cols).  Returns (int32 [n,4] CPU
    tensor, chunk_bytes, out_cols per output).  The chunk size is the largest
    power of two <= 16 bytes that divides every slice length in bytes and whose
    source alignment requirement (min(chunk, 4) bytes) every slice start meets.
    """
    import math

    g = 16
    for sl in slice_lists:
        for s, e in sl:
            if not (0 <= s <= e <= src_cols):
                raise ValueError(f"slice ({s},{e}) outside the source's {src_cols} columns")
            g = math.gcd(g, (e - s) * elem_size)
    stride_bytes = (src_row_stride if src_row_stride is not None else src_cols) * elem_size
    a = math.gcd(16, stride_bytes)
    for sl in slice_lists:
        for s, e in sl:
            if e > s:
                a = math.gcd(a, s * elem_size)
    chunk = max(g, 1)
    if min(chunk, 4) > a:
        chunk = a
    rows_out, out_cols = [], []
    for oid, sl in enumerate(slice_lists):
        dst = 0
        for s, e in sl:
            nbytes = (e - s) * elem_size
            for k in range(0, nbytes, chunk):
                rows_out.append((s * elem_size + k, dst + k, oid, 0))
            dst += nbytes
        out_cols.append(dst // elem_size)
    table = torch.tensor(rows_out, dtype=torch.int32).reshape(-1, 4)
    if table.shape[0] and _lib.is_built():
        # the kernel cannot look at its (device) table: refuse a bad one here, once, on the host
        valid = (ctypes.c_int64 * len(out_cols))(*[c * elem_size for c in out_cols])
        st = _lib.lib().xg_slice_cat_check_table(
            ctypes.c_void_p(table.data_ptr()), table.shape[0], chunk, src_cols * elem_size, valid, len(out_cols)
        )
        _lib.check(st, "xg_slice_cat_check_table")
    return table, chunk, out_cols


# ------------------------------------------------------------- dense / SDPA
_library.define("dense(Tensor x, Tensor weight, bool weight_trans, Tensor? bias, Tensor? residual, str act) -> Tensor")
_library.define("dense_batched(Tensor x, Tensor weight, bool weight_trans, Tensor? bias, Tensor? residual, str act) -> Tensor")
_library.define("dense_at(Tensor a_t, Tensor b, Tensor? residual) -> Tensor")
_library.define("dense_glu(Tensor x, Tensor w_gate, Tensor w_up) -> Tensor")
_library.define("dense_glu_save(Tensor x, Tensor w_gate, Tensor w_up) -> (Tensor, Tensor, Tensor)")
_library.define(
    "dense_fp8(Tensor x_q, Tensor w_q, bool weight_trans, Tensor x_scale, Tensor w_scale, Tensor? bias, str act, ScalarType out_dtype) -> Tensor"
)
_library.define("sdpa(Tensor q, Tensor k, Tensor v, bool is_causal, float scale) -> Tensor")
_library.define("sdpa_lse(Tensor q, Tensor k, Tensor v, bool is_causal, float scale) -> (Tensor, Tensor)")
_library.define(
    "sdpa_bwd(Tensor q, Tensor k, Tensor v, Tensor out, Tensor d_out, Tensor lse, bool is_causal, float scale) -> (Tensor, Tensor, Tensor)"
)
_library.define("sdpa_masked(Tensor q, Tensor k, Tensor v, Tensor? mask, Tensor? scale_t, bool is_causal, float scale) -> Tensor")
_library.define("sdpa_masked_lse(Tensor q, Tensor k, Tensor v, Tensor? mask, Tensor? scale_t, bool is_causal, float scale) -> (Tensor, Tensor)")
_library.define(
    "sdpa_masked_bwd(Tensor q, Tensor k, Tensor v, Tensor out, Tensor d_out, Tensor lse, Tensor? mask, Tensor? scale_t, bool is_causal, "
    "float scale) -> (Tensor, Tensor, Tensor)"
)
_library.define("rope(Tensor x, Tensor cos, Tensor sin) -> Tensor")


def _dense_out_shape(x, weight, weight_trans):
    if x.dim() != 2 or weight.dim() != 2:
        raise ValueError("dense: x and weight must be 2-d")
    k = x.shape[1]
    n, wk = (weight.shape[0], weight.shape[1]) if weight_trans else (weight.shape[1], weight.shape[0])
    if wk != k:
        raise ValueError(f"dense: inner dimensions differ ({k} vs {wk})")
    return x.shape[0], n, k


def _row_major(t):
    """2-D tensor the kernels can read in place: unit last stride, a row stride that is a multiple of 16 bytes and a
    16-byte aligned base.  Anything else (a column slice at an odd offset, a narrow view of a wider buffer whose
    pitch is not a multiple of 16 bytes) is copied, as the reference's modules make such inputs contiguous
    (dense_layer_modules.py:15-16)."""
    per16 = 16 // t.element_size()
    ok = t.stride(-1) == 1 and t.stride(0) >= t.shape[1] and t.stride(0) % per16 == 0 and t.data_ptr() % 16 == 0
    return t if ok else t.contiguous()


def _dense_into(x, weight, weight_trans, bias, residual, act, out):
    """One xg_dense launch writing the contiguous [M, N] tensor `out`."""
    m, n, k = _dense_out_shape(x, weight, weight_trans)
    if act not in _lib.ACT_CODES:
        raise ValueError(f"dense: unknown activation {act!r}")
    if weight.dtype != x.dtype:
        raise TypeError("dense: x and weight must share a dtype")
    x, weight = _row_major(x), _row_major(weight)
    if out.numel() == 0:
        return out
    bias_dt = _code(x.dtype)
    if bias is not None:
        if bias.numel() != n:
            raise ValueError("dense: bias must have N elements")
        bias = bias.contiguous()
        if bias.dtype != x.dtype:
            bias = bias.float()
        bias_dt = _code(bias.dtype)
    ldr = 0
    if residual is not None:
        if tuple(residual.shape) != (m, n) or residual.dtype != x.dtype:
            raise ValueError("dense: residual must be [M, N] in the input dtype")
        residual = _row_major(residual)
        ldr = residual.stride(0)
    st = _lib.lib().xg_dense(
        _ptr(x), _ptr(weight), _ptr(bias), _ptr(residual), _ptr(out), m, n, k, x.stride(0), weight.stride(0), ldr,
        1 if weight_trans else 0, _lib.ACT_CODES[act], _code(x.dtype), bias_dt, _stream(),
    )
    _lib.check(st, "xg_dense")
    return out


def dense_fits(k, n, dtype):
    """What xg_dense takes: static K a multiple of one 16-byte operand load (8 elements of a 16-bit type, 4 of
    fp32), static N a multiple of 8."""
    if dtype not in (torch.bfloat16, torch.float16, torch.float32):
        return False
    per16 = 16 // torch.empty((), dtype=dtype).element_size()
    return isinstance(k, int) and isinstance(n, int) and k > 0 and n > 0 and k % per16 == 0 and n % 8 == 0


def _dense(x, weight, weight_trans, bias, residual, act):
    m, n, _ = _dense_out_shape(x, weight, weight_trans)
    return _dense_into(x, weight, weight_trans, bias, residual, act, torch.empty((m, n), dtype=x.dtype, device=x.device))


MAX_BATCH_PER_LAUNCH = 65535  # gridDim.y of xg_dense_batched


def _dense_batched_shape(x, weight, weight_trans):
    if x.dim() != 3 or weight.dim() != 3 or x.shape[0] != weight.shape[0]:
        raise ValueError("dense_batched: x must be [B, M, K] and weight [B, K, N] (or [B, N, K] with weight_trans)")
    k = x.shape[2]
    wk, n = (weight.shape[2], weight.shape[1]) if weight_trans else (weight.shape[1], weight.shape[2])
    if wk != k:
        raise ValueError("dense_batched: inner dimensions differ")
    return x.shape[0], x.shape[1], n


def _batch_major(t):
    """3-D tensor whose [rows, cols] entries the kernels can read in place (see _row_major) at a batch stride that
    keeps every entry 16-byte aligned."""
    per16 = 16 // t.element_size()
    ok = (
        t.stride(-1) == 1
        and t.stride(1) >= t.shape[2]
        and t.stride(1) % per16 == 0
        and t.stride(0) % per16 == 0
        and t.data_ptr() % 16 == 0
    )
    return t if ok else t.contiguous()


def _dense_batched(x, weight, weight_trans, bias, residual, act):
    """All batch entries in ONE xg_dense_batched launch (the batch index is the second grid axis of the dense kernels).
    bias: [N] shared or [B, N] per batch; residual: [B, M, N]."""
    b, m, n = _dense_batched_shape(x, weight, weight_trans)
    k = x.shape[2]
    if act not in _lib.ACT_CODES:
        raise ValueError(f"dense_batched: unknown activation {act!r}")
    if weight.dtype != x.dtype:
        raise TypeError("dense_batched: x and weight must share a dtype")
    out = torch.empty((b, m, n), dtype=x.dtype, device=x.device)
    if bias is not None and bias.dim() == 2 and bias.shape[0] != b:
        raise ValueError("dense_batched: a 2-D bias must be [B, N]")
    if residual is not None and (tuple(residual.shape) != (b, m, n) or residual.dtype != x.dtype):
        raise ValueError("dense_batched: residual must be [B, M, N] in the input dtype")
    if out.numel() == 0:
        return out
    x, weight = _batch_major(x), _batch_major(weight)
    bias_dt, bias_stride = _code(x.dtype), 0
    if bias is not None:
        if bias.shape[-1] != n:
            raise ValueError("dense_batched: bias must have N elements per entry")
        bias = bias.contiguous()
        if bias.dtype != x.dtype:
            bias = bias.float()
        bias_dt = _code(bias.dtype)
        bias_stride = n if bias.dim() == 2 else 0
    ldr = res_stride = 0
    if residual is not None:
        residual = _batch_major(residual)
        ldr, res_stride = residual.stride(1), residual.stride(0)
    # the batch entry is the second grid axis of the kernels (at most MAX_BATCH_PER_LAUNCH entries a launch): a larger
    # batch goes out in slices, every operand moved on by its batch stride
    esz = x.element_size()
    for b0 in range(0, b, MAX_BATCH_PER_LAUNCH):
        nb = min(MAX_BATCH_PER_LAUNCH, b - b0)

        def at(t, stride, size=esz):
            return t.data_ptr() + b0 * stride * size if t is not None else None

        st = _lib.lib().xg_dense_batched(
            at(x, x.stride(0)), at(weight, weight.stride(0)), at(bias, bias_stride, bias.element_size() if bias is not None else 0),
            at(residual, res_stride), at(out, m * n), nb, m, n, k, x.stride(1), weight.stride(1), ldr,
            x.stride(0), weight.stride(0), bias_stride, res_stride, m * n,
            1 if weight_trans else 0, _lib.ACT_CODES[act], _code(x.dtype), bias_dt, _stream(),
        )
        _lib.check(st, "xg_dense_batched")
    return out


def _dense_batched_meta(x, weight, weight_trans, bias, residual, act):
    b, m, n = _dense_batched_shape(x, weight, weight_trans)
    return torch.empty((b, m, n), dtype=x.dtype, device=x.device)


def _dense_meta(x, weight, weight_trans, bias, residual, act):
    m, n, _ = _dense_out_shape(x, weight, weight_trans)
    return torch.empty((m, n), dtype=x.dtype, device=x.device)


def dense_at_fits(a_shape, b_shape, dtype):
    """What xg_dense_at takes: a_t [K, M], b [K, N], M and N multiples of 8, 16-bit floats; any K."""
    if len(a_shape) != 2 or len(b_shape) != 2 or dtype not in (torch.bfloat16, torch.float16):
        return False
    m, n = a_shape[1], b_shape[1]
    return isinstance(m, int) and isinstance(n, int) and m > 0 and n > 0 and m % 8 == 0 and n % 8 == 0


def _dense_at(a_t, b, residual):
    """a_t.T @ b (+ residual) without materialising the transpose: a_t [K, M], b [K, N] -> [M, N].  The weight gradient
    of a dense layer (gz.T @ x, or x.T @ gz) in one launch of the dense kernel."""
    if a_t.dim() != 2 or b.dim() != 2 or a_t.shape[0] != b.shape[0]:
        raise ValueError("dense_at: a_t must be [K, M] and b [K, N]")
    if a_t.dtype != b.dtype:
        raise TypeError("dense_at: operands must share a dtype")
    k, m = a_t.shape
    n = b.shape[1]
    if not dense_at_fits(tuple(a_t.shape), tuple(b.shape), a_t.dtype):
        raise ValueError("dense_at: needs M % 8 == 0, N % 8 == 0, bf16 or f16")
    out = torch.empty((m, n), dtype=a_t.dtype, device=a_t.device)
    if k == 0:
        return out.zero_() if residual is None else out.copy_(residual)
    a_t, b = _row_major(a_t), _row_major(b)
    ldr = 0
    if residual is not None:
        if tuple(residual.shape) != (m, n) or residual.dtype != a_t.dtype:
            raise ValueError("dense_at: residual must be [M, N] in the operand dtype")
        residual = _row_major(residual)
        ldr = residual.stride(0)
    st = _lib.lib().xg_dense_at(_ptr(a_t), _ptr(b), _ptr(residual), _ptr(out), m, n, k, a_t.stride(0), b.stride(0), ldr, _code(a_t.dtype), _stream())
    _lib.check(st, "xg_dense_at")
    return out


def _dense_at_meta(a_t, b, residual):
    return torch.empty((a_t.shape[1], b.shape[1]), dtype=a_t.dtype, device=a_t.device)


def _dense_fp8(x_q, w_q, weight_trans, x_scale, w_scale, bias, act, out_dtype):
    m, n, k = _dense_out_shape(x_q, w_q, weight_trans)
    if x_q.dtype != torch.float8_e4m3fn or w_q.dtype != torch.float8_e4m3fn:
        raise TypeError("dense_fp8: operands must be float8_e4m3fn")
    if act not in _lib.ACT_CODES:
        raise ValueError(f"dense_fp8: unknown activation {act!r}")
    x_q, w_q = _row_major(x_q), _row_major(w_q)
    x_scale = x_scale.reshape(-1).float().contiguous()
    w_scale = w_scale.reshape(-1).float().contiguous()
    if x_scale.numel() != 1 or w_scale.numel() != n:
        raise ValueError("dense_fp8: x_scale must have 1 element and w_scale N elements")
    out = torch.empty((m, n), dtype=out_dtype, device=x_q.device)
    if out.numel() == 0:
        return out
    bias_dt = XG_F32
    if bias is not None:
        if bias.numel() != n:
            raise ValueError("dense_fp8: bias must have N elements")
        bias = bias.contiguous()
        if bias.dtype != out_dtype:
            bias = bias.float()
        bias_dt = _code(bias.dtype)
    st = _lib.lib().xg_dense_fp8(
        _ptr(x_q), _ptr(w_q), _ptr(x_scale), _ptr(w_scale), _ptr(bias), _ptr(out), m, n, k, x_q.stride(0), w_q.stride(0),
        1 if weight_trans else 0, _lib.ACT_CODES[act], _code(out_dtype), bias_dt, _stream(),
    )
    _lib.check(st, "xg_dense_fp8")
    return out


def _dense_fp8_meta(x_q, w_q, weight_trans, x_scale, w_scale, bias, act, out_dtype):
    m, n, _ = _dense_out_shape(x_q, w_q, weight_trans)
    return torch.empty((m, n), dtype=out_dtype, device=x_q.device)


def _sdpa_check(q, k, v):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("sdpa: q, k, v must be [B, H, S, D]")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[3] or q.shape[1] % max(k.shape[1], 1) != 0:
        raise ValueError("sdpa: inconsistent q/k/v shapes")


def _unit_last(t):
    """A tensor the attention / rotary kernels can read in place: unit last stride, every other stride a multiple of
    16 bytes, 16-byte aligned base (their loads are 16 bytes per lane).  Anything else is copied."""
    per16 = 16 // t.element_size()
    # the offset into the storage stands for the base address (allocations are at least 256-byte aligned), so that the
    # shape-only Meta implementations predict the same layout as the real call
    ok = t.stride(-1) == 1 and all(st % per16 == 0 for st in t.stride()[:-1]) and t.storage_offset() % per16 == 0
    return t if ok else t.contiguous()


def _dense_strides_ok(t):
    """Strides describe a permutation of a contiguous block (no overlap, no gaps)."""
    dims = sorted(((st, sz) for st, sz in zip(t.stride(), t.shape) if sz != 1), key=lambda d: d[0])
    expect = 1
    for st, sz in dims:
        if st != expect:
            return False
        expect *= sz
    return True


def _empty_like_layout(t):
    """Output buffer in the layout of `t` when that layout is dense with a unit last stride (e.g. [B, S, H, D]
    storage viewed as [B, H, S, D]): what follows -- usually transpose(1, 2).reshape(B, S, H*D) -- is then a view."""
    if t.stride(-1) == 1 and _dense_strides_ok(t):
        return torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device=t.device)
    return torch.empty(t.shape, dtype=t.dtype, device=t.device)


# Up to this many query rows per head, against at least this many keys, attention runs on the key-split decode kernel
# (with fewer keys the general kernel's single tile walk is as fast).
_DECODE_ROWS = 32
_DECODE_MIN_KEYS = 512


def _sdpa_run(q, k, v, is_causal, scale, want_lse):
    _sdpa_check(q, k, v)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("sdpa: q, k, v must share a dtype")
    q, k, v = _unit_last(q), _unit_last(k), _unit_last(v)
    B, H, Sq, D = q.shape
    out = _empty_like_layout(q)
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device) if want_lse else None
    if out.numel() == 0:
        return out, lse
    S3 = ctypes.c_int64 * 3
    shape = (B, H, k.shape[1], Sq, k.shape[2], D, S3(*q.stride()[:3]), S3(*k.stride()[:3]), S3(*v.stride()[:3]), S3(*out.stride()[:3]))
    if not is_causal and Sq <= _DECODE_ROWS and k.shape[2] >= _DECODE_MIN_KEYS:
        # a decode step: the keys are split over workgroups; the partial results go through a small workspace
        n_ws = _lib.lib().xg_sdpa_decode_workspace_floats(B, H, k.shape[1], Sq, k.shape[2], D)
        ws = torch.empty((n_ws,), dtype=torch.float32, device=q.device) if n_ws > 0 else None
        st = _lib.lib().xg_sdpa_decode(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), None, None, _code(q.dtype), None, _ptr(ws), n_ws, *shape,
                                       scale, _code(q.dtype), _stream())
        _lib.check(st, "xg_sdpa_decode")
        return out, lse
    tail = (scale, 1 if is_causal else 0, _code(q.dtype), _stream())
    if want_lse:
        _lib.check(_lib.lib().xg_sdpa_lse(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), *shape, *tail), "xg_sdpa_lse")
    else:
        _lib.check(_lib.lib().xg_sdpa(_ptr(q), _ptr(k), _ptr(v), _ptr(out), *shape, *tail), "xg_sdpa")
    return out, lse


def _sdpa(q, k, v, is_causal, scale):
    return _sdpa_run(q, k, v, is_causal, scale, False)[0]


def _sdpa_lse(q, k, v, is_causal, scale):
    """Attention that also returns the natural-log sum of exponentials of every query row ([B, H, Sq] fp32), from
    which the backward kernels recompute the probabilities."""
    return _sdpa_run(q, k, v, is_causal, scale, True)


def _sdpa_bwd(q, k, v, out, d_out, lse, is_causal, scale):
    """Gradients of attention with respect to q, k, v on the flash-style backward kernels: nothing of size
    [Sq, Skv] is stored.  `delta` ([B, H, Sq] fp32, the row sums of d_out * out) is the one temporary."""
    _sdpa_check(q, k, v)
    if out.shape != q.shape or d_out.shape != q.shape or tuple(lse.shape) != tuple(q.shape[:3]):
        raise ValueError("sdpa_bwd: out and d_out must have the shape of q, lse its first three dims")
    if any(t.dtype != q.dtype for t in (k, v, out, d_out)) or lse.dtype != torch.float32:
        raise TypeError("sdpa_bwd: q, k, v, out, d_out must share a dtype; lse is float32")
    q, k, v, out, d_out = (_unit_last(t) for t in (q, k, v, out, d_out))
    lse = lse.contiguous()
    B, H, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    # each gradient in the layout of its tensor: the transpose / reshape that follows in a model's backward is a view
    dq, dk, dv = _empty_like_layout(q), _empty_like_layout(k), _empty_like_layout(v)
    if dq.numel() == 0 or dk.numel() == 0:
        return dq.zero_(), dk.zero_(), dv.zero_()
    delta = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    S3 = ctypes.c_int64 * 3
    st = _lib.lib().xg_sdpa_backward(
        _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(d_out), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(delta), B, H, Hkv, Sq, Skv, D,
        S3(*q.stride()[:3]), S3(*k.stride()[:3]), S3(*v.stride()[:3]), S3(*out.stride()[:3]), S3(*d_out.stride()[:3]),
        S3(*dq.stride()[:3]), S3(*dk.stride()[:3]), S3(*dv.stride()[:3]), scale, 1 if is_causal else 0, _code(q.dtype), _stream(),
    )
    _lib.check(st, "xg_sdpa_backward")
    return dq, dk, dv


def sdpa_mask_fits(mask_shape, q_shape, skv):
    """An additive mask the kernel can index: up to 4-D, last two dims exactly [Sq, Skv], leading dims 1 or the
    batch / head count (broadcast)."""
    if len(mask_shape) < 2 or len(mask_shape) > 4:
        return False
    full = [1] * (4 - len(mask_shape)) + list(mask_shape)
    B, H, Sq = q_shape[0], q_shape[1], q_shape[2]
    return full[2] == Sq and full[3] == skv and full[0] in (1, B) and full[1] in (1, H)


def _mask_operand(mask, q, Skv):
    """The additive mask as the kernels index it: (tensor kept alive, three element strides, dtype code)."""
    S3 = ctypes.c_int64 * 3
    if mask is None:
        return None, None, _code(q.dtype)
    if not sdpa_mask_fits(tuple(mask.shape), tuple(q.shape), Skv):
        raise ValueError("sdpa_masked: the mask must be [Sq, Skv] with up to two leading dims of size 1, B or H")
    if mask.dtype not in (q.dtype, torch.float32):
        if not mask.dtype.is_floating_point:
            raise TypeError("sdpa_masked: the mask must be a floating-point additive mask")
        mask = mask.float()
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    if mask.stride(-1) != 1:
        mask = mask.contiguous()
    strides = S3(*[0 if mask.shape[i] == 1 else mask.stride(i) for i in range(2)], mask.stride(2) if q.shape[2] > 1 else 0)
    return mask, strides, _code(mask.dtype)


def _scale_operand(scale_t):
    if scale_t is None:
        return None
    if scale_t.numel() != 1:
        raise ValueError("sdpa_masked: the scale tensor must have one element")
    return scale_t.reshape(1).to(torch.float32)  # a device op, not a read


def _sdpa_masked_run(q, k, v, mask, scale_t, is_causal, scale, want_lse):
    _sdpa_check(q, k, v)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("sdpa: q, k, v must share a dtype")
    q, k, v = _unit_last(q), _unit_last(k), _unit_last(v)
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    out = _empty_like_layout(q)
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device) if want_lse else None
    if out.numel() == 0:
        return out, lse
    S3 = ctypes.c_int64 * 3
    mask, mask_strides, mask_dt = _mask_operand(mask, q, Skv)
    scale_t = _scale_operand(scale_t)
    if not is_causal and Sq <= _DECODE_ROWS and Skv >= _DECODE_MIN_KEYS:
        n_ws = _lib.lib().xg_sdpa_decode_workspace_floats(B, H, k.shape[1], Sq, Skv, D)
        ws = torch.empty((n_ws,), dtype=torch.float32, device=q.device) if n_ws > 0 else None
        st = _lib.lib().xg_sdpa_decode(
            _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(mask), mask_strides, mask_dt, _ptr(scale_t), _ptr(ws), n_ws, B, H, k.shape[1],
            Sq, Skv, D, S3(*q.stride()[:3]), S3(*k.stride()[:3]), S3(*v.stride()[:3]), S3(*out.stride()[:3]), scale, _code(q.dtype), _stream(),
        )
        _lib.check(st, "xg_sdpa_decode")
        return out, lse
    tail = (mask_strides, mask_dt, _ptr(scale_t), B, H, k.shape[1], Sq, Skv, D, S3(*q.stride()[:3]), S3(*k.stride()[:3]), S3(*v.stride()[:3]),
            S3(*out.stride()[:3]), scale, 1 if is_causal else 0, _code(q.dtype), _stream())
    if want_lse:
        _lib.check(_lib.lib().xg_sdpa_masked_lse(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(mask), *tail), "xg_sdpa_masked_lse")
    else:
        _lib.check(_lib.lib().xg_sdpa_masked(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(mask), *tail), "xg_sdpa_masked")
    return out, lse


def _sdpa_masked(q, k, v, mask, scale_t, is_causal, scale):
    """Attention with an additive mask and / or a scale held in a one-element device tensor (read by the kernel:
    no .item(), no synchronisation)."""
    return _sdpa_masked_run(q, k, v, mask, scale_t, is_causal, scale, False)[0]


def _sdpa_masked_lse(q, k, v, mask, scale_t, is_causal, scale):
    """The same, also returning the log-sum-exp of every query row for the backward kernels."""
    return _sdpa_masked_run(q, k, v, mask, scale_t, is_causal, scale, True)


def _sdpa_masked_bwd(q, k, v, out, d_out, lse, mask, scale_t, is_causal, scale):
    """Gradients of masked / tensor-scaled attention with respect to q, k, v (the mask and the scale tensor get
    none): the backward kernels add the mask to the recomputed scores as the forward did."""
    _sdpa_check(q, k, v)
    if out.shape != q.shape or d_out.shape != q.shape or tuple(lse.shape) != tuple(q.shape[:3]):
        raise ValueError("sdpa_masked_bwd: out and d_out must have the shape of q, lse its first three dims")
    if any(t.dtype != q.dtype for t in (k, v, out, d_out)) or lse.dtype != torch.float32:
        raise TypeError("sdpa_masked_bwd: q, k, v, out, d_out must share a dtype; lse is float32")
    q, k, v, out, d_out = (_unit_last(t) for t in (q, k, v, out, d_out))
    lse = lse.contiguous()
    B, H, Sq, D = q.shape
    Hkv, Skv = k.shape[1], k.shape[2]
    dq, dk, dv = _empty_like_layout(q), _empty_like_layout(k), _empty_like_layout(v)
    if dq.numel() == 0 or dk.numel() == 0:
        return dq.zero_(), dk.zero_(), dv.zero_()
    mask, mask_strides, mask_dt = _mask_operand(mask, q, Skv)
    scale_t = _scale_operand(scale_t)
    delta = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    S3 = ctypes.c_int64 * 3
    st = _lib.lib().xg_sdpa_backward_masked(
        _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(d_out), _ptr(lse), _ptr(mask), mask_strides, mask_dt, _ptr(scale_t), _ptr(dq), _ptr(dk),
        _ptr(dv), _ptr(delta), B, H, Hkv, Sq, Skv, D, S3(*q.stride()[:3]), S3(*k.stride()[:3]), S3(*v.stride()[:3]), S3(*out.stride()[:3]),
        S3(*d_out.stride()[:3]), S3(*dq.stride()[:3]), S3(*dk.stride()[:3]), S3(*dv.stride()[:3]), scale, 1 if is_causal else 0,
        _code(q.dtype), _stream(),
    )
    _lib.check(st, "xg_sdpa_backward_masked")
    return dq, dk, dv


def _sdpa_masked_meta(q, k, v, mask, scale_t, is_causal, scale):
    _sdpa_check(q, k, v)
    return _empty_like_layout(_unit_last(q))


def _sdpa_masked_lse_meta(q, k, v, mask, scale_t, is_causal, scale):
    _sdpa_check(q, k, v)
    return _empty_like_layout(_unit_last(q)), torch.empty(tuple(q.shape[:3]), dtype=torch.float32, device=q.device)


def _sdpa_masked_bwd_meta(q, k, v, out, d_out, lse, mask, scale_t, is_causal, scale):
    _sdpa_check(q, k, v)
    return tuple(_empty_like_layout(_unit_last(t)) for t in (q, k, v))


def _sdpa_meta(q, k, v, is_causal, scale):
    _sdpa_check(q, k, v)
    return _empty_like_layout(_unit_last(q))


def _sdpa_lse_meta(q, k, v, is_causal, scale):
    _sdpa_check(q, k, v)
    return _empty_like_layout(_unit_last(q)), torch.empty(tuple(q.shape[:3]), dtype=torch.float32, device=q.device)


def _sdpa_bwd_meta(q, k, v, out, d_out, lse, is_causal, scale):
    _sdpa_check(q, k, v)
    return tuple(_empty_like_layout(_unit_last(t)) for t in (q, k, v))


def _rope_check(x, cos, sin):
    if x.dim() != 4:
        raise ValueError("rope: x must be [B, H, S, D]")
    S, D = x.shape[2], x.shape[3]
    if D % 16 != 0:
        raise ValueError("rope: head dim must be a multiple of 16")
    for t in (cos, sin):
        rows_ok = t.dim() == 1 or (t.dim() >= 2 and t.shape[-2] in (1, S))
        if t.dim() < 1 or t.shape[-1] != D or not rows_ok or any(d != 1 for d in t.shape[:-2]):
            raise ValueError("rope: cos / sin must be [S, D] tables or one row [D] (leading dims of size 1 allowed)")
    if cos.shape != sin.shape:
        raise ValueError("rope: cos and sin must have the same shape")
    if cos.dtype != sin.dtype or cos.dtype not in (x.dtype, torch.float32):
        raise TypeError("rope: cos / sin must share a dtype, that of x or float32")


def _rope(x, cos, sin):
    _rope_check(x, cos, sin)
    x = _unit_last(x)
    B, H, S, D = x.shape
    out = _empty_like_layout(x)
    if out.numel() == 0:
        return out
    cos2, sin2 = cos.reshape(-1, D), sin.reshape(-1, D)
    if cos2.shape[0] != S:  # one row for every position: a table of S equal rows (S is 1 in a decode step: a view)
        cos2, sin2 = cos2.expand(S, D), sin2.expand(S, D)
    if cos2.stride(1) != 1 or sin2.stride() != cos2.stride() or (S > 1 and cos2.stride(0) < D):
        cos2, sin2 = cos2.contiguous(), sin2.contiguous()
    S3 = ctypes.c_int64 * 3
    st = _lib.lib().xg_rope(
        _ptr(x), _ptr(cos2), _ptr(sin2), _ptr(out), B, H, S, D, S3(*x.stride()[:3]), S3(*out.stride()[:3]), max(cos2.stride(0), D),
        _code(x.dtype), _code(cos2.dtype), _stream(),
    )
    _lib.check(st, "xg_rope")
    return out


def _rope_meta(x, cos, sin):
    _rope_check(x, cos, sin)
    return _empty_like_layout(_unit_last(x))


_GLU_OPERAND_LIMIT = 2**31 - 1


def dense_glu_fits(x_shape, w_shape, dtype):
    """What the gated kernel takes: 2-D x [M, K], two [N, K] weights, K a multiple of 64, N of 8, 16-bit floats."""
    if len(x_shape) != 2 or len(w_shape) != 2 or dtype not in (torch.bfloat16, torch.float16):
        return False
    m, k, n = x_shape[0], x_shape[1], w_shape[0]
    ints = all(isinstance(d, int) for d in (k, *w_shape))  # the row count may be symbolic
    if not (ints and w_shape[1] == k and k % 64 == 0 and n % 8 == 0 and k > 0 and n > 0):
        return False
    # the gated kernel addresses each operand with a 31-bit byte offset and has no other variant: operands known to
    # be 2 GiB or more stay two dense layers and a gate kernel (a symbolic row count is decided per call, see _dense_glu)
    m_ok = not isinstance(m, int) or m * k * 2 < _GLU_OPERAND_LIMIT
    return m_ok and n * k * 2 < _GLU_OPERAND_LIMIT


def _dense_glu_run(x, w_gate, w_up, save):
    """silu(x @ w_gate.T) * (x @ w_up.T) in one launch; weights are [N, K] (torch.nn.Linear layout).  save: also
    return the two rounded projections the gate was computed from."""
    if w_gate.shape != w_up.shape or w_gate.dtype != x.dtype or w_up.dtype != x.dtype:
        raise ValueError("dense_glu: the two weights must share shape and dtype with each other and with x")
    if not dense_glu_fits(tuple(x.shape), tuple(w_gate.shape), x.dtype):
        raise ValueError("dense_glu: needs x [M, K], weights [N, K], K % 64 == 0, N % 8 == 0, bf16 or f16")
    x, w_gate, w_up = _row_major(x), _row_major(w_gate), _row_major(w_up)
    if w_up.stride(0) != w_gate.stride(0):
        w_gate, w_up = w_gate.contiguous(), w_up.contiguous()
    m, k = x.shape
    n = w_gate.shape[0]
    if m * x.stride(0) * 2 >= _GLU_OPERAND_LIMIT or n * w_gate.stride(0) * 2 >= _GLU_OPERAND_LIMIT:
        # a row count that was symbolic at match time turned out too large for the gated kernel's 31-bit operand
        # offsets: the same result, bit for bit, from two dense launches and the gate kernel
        gate, up = _dense(x, w_gate, True, None, None, "none"), _dense(x, w_up, True, None, None, "none")
        return _silu_mul2(gate, up), gate, up
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    gate = torch.empty((m, n), dtype=x.dtype, device=x.device) if save else None
    up = torch.empty((m, n), dtype=x.dtype, device=x.device) if save else None
    if out.numel() == 0:
        return out, gate, up
    args = (m, n, k, x.stride(0), w_gate.stride(0), _code(x.dtype), _stream())
    if save:
        _lib.check(_lib.lib().xg_dense_glu_save(_ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(out), _ptr(gate), _ptr(up), *args), "xg_dense_glu_save")
    else:
        _lib.check(_lib.lib().xg_dense_glu(_ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(out), *args), "xg_dense_glu")
    return out, gate, up


def _dense_glu(x, w_gate, w_up):
    return _dense_glu_run(x, w_gate, w_up, False)[0]


def _dense_glu_save(x, w_gate, w_up):
    return _dense_glu_run(x, w_gate, w_up, True)


def _dense_glu_save_meta(x, w_gate, w_up):
    shape = (x.shape[0], w_gate.shape[0])
    return tuple(torch.empty(shape, dtype=x.dtype, device=x.device) for _ in range(3))


_library.impl("dense", _dense, "CUDA")
_library.impl("dense_glu", _dense_glu, "CUDA")
_library.impl("dense_glu_save", _dense_glu_save, "CUDA")
_library.impl("dense_glu_save", _dense_glu_save_meta, "Meta")
_library.impl("dense_glu", lambda x, w_gate, w_up: torch.empty((x.shape[0], w_gate.shape[0]), dtype=x.dtype, device=x.device), "Meta")
_library.impl("dense", _dense_meta, "Meta")
_library.impl("dense_at", _dense_at, "CUDA")
_library.impl("dense_at", _dense_at_meta, "Meta")
_library.impl("dense_batched", _dense_batched, "CUDA")
_library.impl("dense_batched", _dense_batched_meta, "Meta")
_library.impl("dense_fp8", _dense_fp8, "CUDA")
_library.impl("dense_fp8", _dense_fp8_meta, "Meta")
_library.impl("sdpa", _sdpa, "CUDA")
_library.impl("sdpa", _sdpa_meta, "Meta")
_library.impl("sdpa_lse", _sdpa_lse, "CUDA")
_library.impl("sdpa_lse", _sdpa_lse_meta, "Meta")
_library.impl("sdpa_bwd", _sdpa_bwd, "CUDA")
_library.impl("sdpa_bwd", _sdpa_bwd_meta, "Meta")
_library.impl("sdpa_masked", _sdpa_masked, "CUDA")
_library.impl("sdpa_masked", _sdpa_masked_meta, "Meta")
_library.impl("sdpa_masked_lse", _sdpa_masked_lse, "CUDA")
_library.impl("sdpa_masked_lse", _sdpa_masked_lse_meta, "Meta")
_library.impl("sdpa_masked_bwd", _sdpa_masked_bwd, "CUDA")
_library.impl("sdpa_masked_bwd", _sdpa_masked_bwd_meta, "Meta")
_library.impl("rope", _rope, "CUDA")
_library.impl("rope", _rope_meta, "Meta")


# ------------------------------------------------------------- training
def enable_autograd():
    """Register the backward formulas of the ops that may appear in training graphs (xpu_graph_amd/autograd.py).
    Done on demand -- by a backend constructed with is_training=True -- because an op with a Python autograd
    formula pays a few microseconds of dispatch on every call, which inference-only processes need not."""
    from . import autograd as _autograd

    _autograd.register()
