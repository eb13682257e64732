"""Modules the structure patterns substitute on the mi355x target.  Signatures
are the reference's (passes/patterns/targets/mlu/structure_replacements/
__init__.py:27-179, dense_layer_modules.py:4-68, norm_modules.py:4-21); bodies
call `torch.ops.xpu_ops.*`, i.e. the HIP kernels, and nothing else."""
import torch
from torch._subclasses.fake_tensor import FakeTensor

from ..... import ops as _xops

_DENSE_DTYPES = (torch.bfloat16, torch.float16)


class RMSNormModule(torch.nn.Module):
    def forward(self, inputs, weight, eps):
        return torch.ops.xpu_ops.rms_norm(inputs, weight, eps)


class LayerNormModule(torch.nn.Module):
    def forward(self, inputs, weight, bias, eps):
        return torch.ops.xpu_ops.layer_norm(inputs, weight, bias, eps)


class _SliceTables:
    """Per-(slice list, source layout, device) cache of device-resident chunk tables,
    so the steady state does no host work beyond a dict lookup."""

    def __init__(self):
        self._cache = {}

    def get(self, src, slice_lists):
        if isinstance(src, FakeTensor):
            # shape propagation only (sizes and strides may be symbolic): the op's output shape depends on the
            # slice widths alone, so any table stands in
            out_cols = [sum(e - s for s, e in sl) for sl in slice_lists]
            return torch.empty((1, 4), dtype=torch.int32, device=src.device), 4, out_cols
        key = (tuple(tuple(map(tuple, sl)) for sl in slice_lists), src.shape[1], src.stride(0), src.element_size(), str(src.device))
        hit = self._cache.get(key)
        if hit is None:
            table, chunk, out_cols = _xops.build_slice_table(slice_lists, src.shape[1], src.element_size(), src.stride(0))
            hit = (table.to(src.device), chunk, out_cols)
            self._cache[key] = hit
        return hit

    def __getstate__(self):
        return {}

    def __setstate__(self, state):
        self._cache = {}


def _check_2d(t):
    if t.dim() != 2:
        raise NotImplementedError("input must be 2d")
    if t.stride(1) != 1:
        t = t.contiguous()
    return t


class FuseSliceCatSameInputModule(torch.nn.Module):
    """forward(input2d, [(start, end), ...]) -> [rows, sum(end - start)]"""

    def __init__(self):
        super().__init__()
        self._tables = _SliceTables()

    def forward(self, input_tensor, slices):
        src = _check_2d(input_tensor)
        table, chunk, out_cols = self._tables.get(src, [slices])
        return torch.ops.xpu_ops.slice_cat(src, table, chunk, out_cols[0])


class FuseSliceCatSameInputModule_v2(torch.nn.Module):
    """Built with the static table of all slice lists; forward returns one tensor per list, from ONE launch."""

    def __init__(self, many_slices):
        super().__init__()
        self.many_slices = [list(map(tuple, sl)) for sl in many_slices]
        self._tables = _SliceTables()

    def forward(self, input_tensor, many_slices=None):
        src = _check_2d(input_tensor)
        lists = self.many_slices
        step = _xops._lib.SLICE_CAT_MAX_OUTS
        outs = []
        for lo in range(0, len(lists), step):
            part = lists[lo : lo + step]
            table, chunk, out_cols = self._tables.get(src, part)
            outs += torch.ops.xpu_ops.slice_cat_multi(src, table, chunk, out_cols)
        return outs


class FuseSliceModule(torch.nn.Module):
    """Built with the start columns of equally wide slices of ONE source (last dim); forward(input, slice_len) ->
    [n_slices, *input.shape[:-1], slice_len], slab k = input[..., start_k : start_k + slice_len]
    (reference FuseSliceModule, structure_replacements/__init__.py:21-47).  One launch per 32 slices, every slab
    written straight into the one result buffer."""

    def __init__(self, slices_index):
        super().__init__()
        self.slices_index = [int(s) for s in slices_index]
        self._tables = _SliceTables()

    def forward(self, input_tensor, slice_len):
        lead = list(input_tensor.shape[:-1])
        src = input_tensor if input_tensor.dim() == 2 else input_tensor.reshape(-1, input_tensor.shape[-1])
        src = _check_2d(src)
        step = _xops._lib.SLICE_CAT_MAX_OUTS
        tables, chunks = [], []
        for lo in range(0, len(self.slices_index), step):
            part = [[(s, s + slice_len)] for s in self.slices_index[lo : lo + step]]
            table, chunk, _ = self._tables.get(src, part)
            tables.append(table)
            chunks.append(chunk)
        out = torch.ops.xpu_ops.slice_stack(src, tables, chunks, slice_len, len(self.slices_index))
        return out.view([len(self.slices_index)] + lead + [slice_len])


class ComboSumModule(torch.nn.Module):
    """forward([3-D tensors], [dim]) -> [2-D sums]; one launch for all jobs."""

    def forward(self, input_list, dim):
        return torch.ops.xpu_ops.combo_sum(list(input_list), dim[0])


class DenseLayerModule(torch.nn.Module):
    """forward(inputs, weight, weight_trans, bias | None, act) -> act(inputs @ W(+T) + bias).
    A 1-D (or [1, N]) bias is a bias; a 2-D bias is a residual added before the activation."""

    def __init__(self, fast_act=False):
        super().__init__()
        self.fast_act = fast_act

    def forward(self, inputs, weight, weight_trans, bias, act):
        n = weight.shape[-2] if weight_trans else weight.shape[-1]
        m = inputs.shape[0]
        residual = None
        if bias is not None:
            if bias.dim() == 2 and bias.shape[0] == 1:
                bias = bias.reshape(-1)
            if bias.dim() == 1:
                if bias.shape[0] != n:
                    bias = bias.broadcast_to((n,)).contiguous()
            else:
                residual = bias if tuple(bias.shape) == (m, n) else bias.broadcast_to((m, n)).contiguous()
                bias = None
        if act != "none" and torch.is_grad_enabled() and any(
            t is not None and t.requires_grad for t in (inputs, weight, bias, residual)
        ):
            # a graph that will be differentiated keeps the pre-activation, as eager does: the backward is then one
            # pass over it (xpu_ops::act_bwd) instead of a second product and a chain of fp32 Aten formulas
            z = torch.ops.xpu_ops.dense(inputs, weight, weight_trans, bias, residual, "none")
            return torch.ops.xpu_ops.act(z, act)
        return torch.ops.xpu_ops.dense(inputs, weight, weight_trans, bias, residual, act)


def can_fuse_custom_denselayer(inputs, weight, weight_trans, bias, act_str):
    """Match-time veto (arguments are FakeTensors): what the MFMA kernels cannot take stays in Aten.  bf16 / f16
    (32x32x16 MFMA) and fp32 (32x32x2 fp32 MFMA, the dtype of the reference's own dense-layer tests,
    tests/mlu/test_custom_denselayer.py:11)."""
    if act_str not in ("none", "relu", "gelu", "silu", "sigmoid"):
        return False
    if inputs.dtype not in (*_DENSE_DTYPES, torch.float32) or weight.dtype != inputs.dtype:
        return False
    if inputs.dim() != 2 or weight.dim() != 2:
        return False
    if bias is not None and (bias.dtype != inputs.dtype or bias.dim() > 2):
        return False
    k = inputs.shape[1]
    n = weight.shape[0] if weight_trans else weight.shape[1]
    return _xops.dense_fits(k, n, inputs.dtype)


class BatchDenseLayerModule(torch.nn.Module):
    """forward(inputs [B,M,K], weight [B,K,N] | [B,N,K], weight_trans, bias | None, act): a bias of the output's
    shape is a residual, anything else must broadcast to [B, 1, N]
    (reference targets/mlu/structure_replacements/dense_layer_modules.py:71-111)."""

    def forward(self, inputs, weight, weight_trans, bias, act):
        b, m, _ = inputs.shape
        n = weight.shape[-2] if weight_trans else weight.shape[-1]
        residual = None
        if bias is not None:
            if tuple(bias.shape) == (b, m, n) and m != 1:
                residual, bias = bias, None
            elif bias.dim() == 1 or all(d == 1 for d in bias.shape[:-1]):
                bias = bias.reshape(-1)
                if bias.shape[0] != n:
                    bias = bias.broadcast_to((n,)).contiguous()
            else:
                bias = bias.broadcast_to((b, 1, n)).reshape(b, n)
        return torch.ops.xpu_ops.dense_batched(inputs, weight, weight_trans, bias, residual, act)


def can_fuse_custom_batch_denselayer(inputs, weight, weight_trans, bias, act_str):
    """Match-time veto (FakeTensors): 3-D operands of a 16-bit type with static, 8-aligned K and N."""
    if act_str not in ("none", "relu", "gelu", "silu", "sigmoid"):
        return False
    if inputs.dim() != 3 or weight.dim() != 3 or inputs.dtype not in _DENSE_DTYPES or weight.dtype != inputs.dtype:
        return False
    dims = (*inputs.shape, *weight.shape)
    if not all(isinstance(d, int) for d in dims) or inputs.shape[0] != weight.shape[0]:
        return False
    k = inputs.shape[2]
    n = weight.shape[1] if weight_trans else weight.shape[2]
    if bias is not None:
        b, m = inputs.shape[0], inputs.shape[1]
        if bias.dtype != inputs.dtype or not all(isinstance(d, int) for d in bias.shape):
            return False
        try:
            if tuple(torch.broadcast_shapes(tuple(bias.shape), (b, m, n))) != (b, m, n):
                return False
        except RuntimeError:
            return False
        if tuple(bias.shape) != (b, m, n) and bias.dim() == 3 and bias.shape[1] != 1:
            return False  # varies along M without being a full residual
        if bias.dim() == 2 and bias.shape[0] != 1:
            return False  # [M, N]-shaped bias: neither per-batch nor shared
    return k % 8 == 0 and n % 8 == 0 and k > 0 and n > 0


def get_structure_replacements(config):
    return {
        "CustomRMSNorm": RMSNormModule,
        "CustomLayerNorm": LayerNormModule,
        "FusedCatSlice": FuseSliceCatSameInputModule,
        "FusedSliceStackSum": FuseSliceCatSameInputModule,
        "FusedMultipleSliceCat": FuseSliceCatSameInputModule_v2,
        "FusedSlice": FuseSliceModule,
        "ComboSum3dInp": ComboSumModule,
        "CustomDenseLayer": (DenseLayerModule, can_fuse_custom_denselayer),
        "CustomBatchDenseLayer": (BatchDenseLayerModule, can_fuse_custom_batch_denselayer),
    }
