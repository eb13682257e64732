"""All twenty eager spellings of attention that the reference pins for FusedSDPA
(reference tests/common/test_fuse_sdpa.py:580-601 lists them, :14-560 defines them), on the default path, at the
reference's own sizes and dtype (fp16, heads 32, sequence 38, head size 64, batch 1 / 2 / 4, :563-575) and with its
comparison (`is_similar`, rtol = atol = 1e-2): the matcher has to fire on each and the result has to follow eager.

The forms are written here from their mathematics, grouped by what varies: how the scale enters (divide, multiply,
tensor, clamped tensor, pre-scaled query, none), whether a mask is added or subtracted, an identity dropout (p = 0)
in three spellings, a detour of the softmax through fp32, operands that arrive as [B, S, H, E] and are permuted, 3-D
bmm operands, and the transposed, contiguous output of the decoder models."""
import math

import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs, skip_xpu_graph_cache

HALF = torch.half
HEADS, SEQ, E = 32, 38, 64


def bhse(b):  # operands as [B, H, S, E]
    return tuple(torch.randn(b, HEADS, SEQ, E, dtype=HALF) for _ in range(3))


def bshe(b):  # operands as [B, S, H, E]: the function permutes them itself
    return tuple(torch.randn(b, SEQ, HEADS, E, dtype=HALF) for _ in range(3))


def hse(b):  # 3-D operands of a bmm
    return tuple(torch.randn(HEADS, SEQ, E, dtype=HALF) for _ in range(3))


def full_mask(b):
    return torch.randn(b, HEADS, SEQ, SEQ, dtype=HALF)


def heads_first(*ts):
    return tuple(t.permute(0, 2, 1, 3) for t in ts)


def scores(q, k):
    return torch.matmul(q, k.transpose(-2, -1))


# ---- scale enters by a division / a multiplication; python number, tensor, clamped tensor
def divide_by_number(q, k, v, inv):
    return scores(q, k).div(inv).softmax(dim=-1).matmul(v)


def divide_by_clamped_tensor(q, k, v, inv):
    return scores(q, k).div(torch.clamp(torch.tensor([inv], dtype=q.dtype, device=q.device), 0, 20)).softmax(dim=-1).matmul(v)


def multiply_by_number(q, k, v, s):
    return scores(q, k).mul(s).softmax(dim=-1).matmul(v)


def divide_then_identity_dropout(q, k, v, inv, p=0.0):
    return F.dropout(scores(q, k).div(inv).softmax(dim=-1), p=p).matmul(v)


def multiply_then_identity_dropout(q, k, v, s, p=0.0):
    return F.dropout(scores(q, k).mul(s).softmax(dim=-1), p=p).matmul(v)


# ---- operator spelling with 1 / sqrt(E); mask added or subtracted; aten.dropout with train=True and p = 0
def root_scale_plus_mask(q, k, v, m):
    return torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(q.size(-1)) + m, dim=-1) @ v


def root_scale(q, k, v):
    return torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(q.size(-1)), dim=-1) @ v


def root_scale_plus_mask_dropout(q, k, v, m, p=0.0):
    w = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(q.size(-1)) + m, dim=-1)
    return torch.dropout(w, p, True) @ v


def root_scale_minus_mask_dropout(q, k, v, m, p=0.0):
    w = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(q.size(-1)) - m, dim=-1)
    return torch.dropout(w, p, True) @ v


# ---- [B, S, H, E] operands permuted inside, softmax through fp32 and back to half
def permuted_fp32_softmax(query, key, value, p=None):
    q, k, v = heads_first(query, key, value)
    w = torch.softmax((q @ k.transpose(-2, -1) / math.sqrt(q.size(-1))).to(torch.float32), dim=-1)
    if p is not None:
        w = torch.dropout(w, p, True)
    return w.to(v.dtype) @ v


def permuted_prescaled_query(query, key, value, p=None):
    q, k, v = heads_first(query, key, value)
    w = torch.softmax(((q / math.sqrt(q.size(-1))) @ k.transpose(-2, -1)).to(torch.float32), dim=-1)
    if p is not None:
        w = torch.dropout(w, p, True)
    return w.to(v.dtype) @ v


def permuted_divide(query, key, value, inv):
    q, k, v = heads_first(query, key, value)
    return scores(q, k).div(inv).softmax(dim=-1).matmul(v)


def permuted_divide_dropout(query, key, value, inv, p=0.0):
    q, k, v = heads_first(query, key, value)
    return F.dropout(scores(q, k).div(inv).softmax(dim=-1), p=p).matmul(v)


# ---- 3-D operands, no scale
def bmm_no_scale(q, k, v, p=0.0):
    w = F.dropout(torch.bmm(q, k.transpose(1, 2)).softmax(dim=-1), p=p)
    return torch.bmm(w, v)


# ---- decoder models: softmax(dtype=fp32) cast back, inference dropout, output handed on as [B, S, H, E]
def decoder(q, k, v):
    w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(q.size(-1))
    w = F.dropout(F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype), p=0.0, training=False)
    return torch.matmul(w, v).transpose(1, 2).contiguous()


def decoder_with_sliced_mask(q, k, v, mask):
    w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(q.size(-1))
    w = w + mask[:, :, :, : k.shape[-2]]
    w = F.dropout(F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype), p=0.0, training=False)
    return torch.matmul(w, v).transpose(1, 2).contiguous()


def decoder_in_place_scale(q, k, v, mask):
    w = q @ k.transpose(-1, -2)
    w /= math.sqrt(q.size(-1))
    return F.softmax(w + mask, dim=-1, dtype=q.dtype) @ v


ROOT, INV = math.sqrt(E), 1.0 / math.sqrt(E)
# (name in the reference's list, function, operand layout, further arguments as a function of the batch size)
FORMS = [
    ("tensor_scale", divide_by_number, bhse, lambda b: (torch.Tensor([ROOT]).to(HALF),)),
    ("transformer_1", decoder, bhse, lambda b: ()),
    ("transformer_2", decoder_with_sliced_mask, bhse, lambda b: (full_mask(b),)),
    ("transformer_3", decoder_in_place_scale, bhse, lambda b: (full_mask(b),)),
    ("1", divide_by_number, bhse, lambda b: (ROOT,)),
    ("1_1", divide_by_clamped_tensor, bhse, lambda b: (ROOT,)),
    ("2", multiply_by_number, bhse, lambda b: (INV,)),
    ("3", divide_then_identity_dropout, bhse, lambda b: (ROOT,)),
    ("4", multiply_then_identity_dropout, bhse, lambda b: (INV,)),
    ("5", root_scale_plus_mask, bhse, lambda b: (full_mask(b),)),
    ("5_1", root_scale, bhse, lambda b: ()),
    ("6", root_scale_plus_mask_dropout, bhse, lambda b: (full_mask(b), 0.0)),
    ("6_1", root_scale_minus_mask_dropout, bhse, lambda b: (full_mask(b), 0.0)),
    ("7", permuted_fp32_softmax, bshe, lambda b: (0.0,)),
    ("8", permuted_fp32_softmax, bshe, lambda b: ()),
    ("9", permuted_prescaled_query, bshe, lambda b: (0.0,)),
    ("10", permuted_prescaled_query, bshe, lambda b: ()),
    ("11", permuted_divide, bshe, lambda b: (ROOT,)),
    ("12", permuted_divide_dropout, bshe, lambda b: (ROOT,)),
    ("13", bmm_no_scale, hse, lambda b: ()),
]


@pytest.fixture(scope="module")
def backend():
    return XpuGraph(
        XpuGraphConfig(is_training=False, freeze=False, constant_folding=True, folding_freezed_params=False, opt_level=OptLevel.level2)
    )


def test_the_list_is_the_references():
    assert len(FORMS) == 20 and len({name for name, *_ in FORMS}) == 20


@pytest.mark.parametrize("name,fn,layout,extra", FORMS, ids=[f[0] for f in FORMS])
def test_reference_sdpa_form(caplog, backend, name, fn, layout, extra):
    torch.manual_seed(len(name) + 7)
    with need_xpu_graph_logs(), skip_xpu_graph_cache(backend):
        compiled = torch.compile(fn, backend=backend, dynamic=None)
        for b in (1, 2, 4):
            args = layout(b) + extra(b)
            got, want = compiled(*args), fn(*args)
            if not is_similar(got.float(), want.float()):
                # unscaled fp16 scores (standard deviation 8) make eager's own rounding of them visible: there the
                # compiled result has to be at least as close to the fp32 evaluation as eager is
                exact = fn(*(a.float() if torch.is_tensor(a) else a for a in args))
                err_got, err_eager = (got.float() - exact).abs().max().item(), (want.float() - exact).abs().max().item()
                assert name == "13" and err_got <= err_eager, (name, b, err_got, err_eager)
    assert "Pattern.FusedSDPA changed graph" in caplog.text
    if name == "tensor_scale":
        assert "Unwrap scale " in caplog.text
