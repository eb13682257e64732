"""Norm recognisers on the default (CPU, target=none) path: every accepted
spelling fires the pattern and the compiled result equals eager.  Variants and
dtype mixes follow the reference's tests/common/test_fuse_rmsnorm.py:20-123 and
tests/common/test_fuse_layernorm.py:20-140."""
import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs

f32, f16, bf16 = torch.float32, torch.float16, torch.bfloat16


def rms_div_sqrt(x, w):
    return x / torch.sqrt(torch.mean(torch.square(x), dim=-1, keepdim=True) + 1e-6) * w


def rms_rsqrt_weight_first(x, w):
    return w * (x * torch.rsqrt(torch.mean(x**2, dim=-1, keepdim=True) + 1e-6))


def rms_pow_half_noweight(x, w):
    return x / ((x * x).mean(dim=-1, keepdim=True) + 1e-3) ** 0.5


def rms_upcast_input(x, w):
    return rms_div_sqrt(x.to(f32), w).to(x.dtype)


def rms_upcast_weight(x, w):
    return rms_div_sqrt(x, w.to(f32)).to(x.dtype)


def rms_baseline_c1(x, w):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w


def rms_library(x, w):
    return F.rms_norm(x, (x.shape[-1],), w, 1e-6)


@pytest.fixture(scope="module")
def backend():
    return XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2))


@pytest.mark.parametrize(
    "fn,xdt,wdt",
    [
        (rms_div_sqrt, f32, f32),
        (rms_div_sqrt, f16, f32),
        (rms_rsqrt_weight_first, f16, f16),
        (rms_pow_half_noweight, f32, f32),
        (rms_upcast_input, f32, f16),
        (rms_upcast_input, f32, bf16),
        (rms_upcast_input, f16, f16),
        (rms_upcast_input, f16, f32),
        (rms_upcast_weight, f32, f16),
        (rms_upcast_weight, f16, f16),
        (rms_baseline_c1, f32, f32),
        (rms_library, f32, f32),
    ],
)
@pytest.mark.parametrize("dynamic", [False, True])
def test_rmsnorm_spellings(caplog, backend, fn, xdt, wdt, dynamic):
    torch.manual_seed(0)
    x = torch.randn(8, 1024, dtype=xdt)
    w = torch.randn(1024, dtype=wdt)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend, dynamic=dynamic)(x, w)
    assert is_similar(got.float(), fn(x, w).float())
    assert got.dtype == fn(x, w).dtype
    assert "Pattern.FusedRMSNorm changed graph" in caplog.text
    if fn is rms_upcast_input and xdt != f32:
        assert "Pattern.RemoveRMSNormCast" in caplog.text
    if fn is rms_upcast_weight and wdt != f32:
        assert "Pattern.RemoveRMSNormCast" in caplog.text


def not_rms_mean_over_rows(x, w):
    return x * torch.rsqrt(x.pow(2).mean(0, keepdim=True) + 1e-6) * w


def not_rms_shared_rsqrt(x, w):
    r = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
    return x * r * w + r  # the rsqrt has a second user: fusing would lose it


@pytest.mark.parametrize("fn", [not_rms_mean_over_rows, not_rms_shared_rsqrt])
def test_rmsnorm_must_not_fire(caplog, backend, fn):
    x, w = torch.randn(16, 16), torch.randn(16)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend)(x, w)
    torch.testing.assert_close(got, fn(x, w))
    assert "Pattern.FusedRMSNorm changed graph" not in caplog.text


def ln_full(x, w, b):
    m = torch.mean(x, dim=-1, keepdim=True)
    v = torch.var(x, dim=-1, keepdim=True, unbiased=False)
    return w * ((x - m) / ((v + 1e-6) ** 0.5)) + b


def ln_bias_only(x, w, b):
    m = torch.mean(x, dim=-1, keepdim=True)
    v = torch.var(x, dim=-1, keepdim=True, unbiased=False)
    return b + (x - m) * torch.rsqrt(1e-6 + v)


def ln_plain(x, w, b):
    m = torch.mean(x, dim=-1, keepdim=True)
    v = torch.var(x, dim=-1, keepdim=True, correction=0)
    return (x - m) / torch.sqrt(v + 1e-5)


def ln_weight_only(x, w, b):
    m = torch.mean(x, dim=-1, keepdim=True)
    v = torch.var(x, dim=-1, keepdim=True, correction=0)
    return w * ((x - m) * ((v + 1e-5) ** (-0.5)))


def ln_upcast_input(x, w, b):
    return ln_full(x.to(f32), w, b).to(x.dtype)


def ln_upcast_params(x, w, b):
    return ln_full(x, w.to(f32), b.to(f32)).to(x.dtype)


@pytest.mark.parametrize(
    "fn,xdt,wdt,bdt",
    [
        (ln_full, f32, f32, f32),
        (ln_full, f16, f32, f32),
        (ln_full, f16, f32, f16),
        (ln_bias_only, f32, f32, f32),
        (ln_plain, f32, f32, f32),
        (ln_weight_only, f16, f16, f16),
        (ln_upcast_input, f16, f16, f16),
        (ln_upcast_input, f16, f32, f32),
        (ln_upcast_input, bf16, f32, bf16),
        (ln_upcast_params, f32, f16, f16),
        (ln_upcast_params, f16, f16, f16),
    ],
)
@pytest.mark.parametrize("dynamic", [False, True])
def test_layernorm_spellings(caplog, backend, fn, xdt, wdt, bdt, dynamic):
    torch.manual_seed(0)
    x = torch.randn(8, 1024, dtype=xdt)
    w = torch.randn(1024, dtype=wdt)
    b = torch.randn(1024, dtype=bdt)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend, dynamic=dynamic)(x, w, b)
    want = fn(x, w, b)
    assert got.dtype == want.dtype
    assert is_similar(got.float(), want.float(), rtol=0.02, atol=0.02)
    assert "Pattern.FusedLayerNorm changed graph" in caplog.text
    if fn in (ln_upcast_input, ln_upcast_params) and (xdt, wdt, bdt) != (f32, f32, f32):
        assert "Pattern.RemoveLayerNormCast" in caplog.text


def test_layernorm_biased_variance_not_matched(caplog, backend):
    def fn(x):
        m = x.mean(-1, keepdim=True)
        return (x - m) * torch.rsqrt(x.var(-1, keepdim=True) + 1e-5)  # unbiased variance is not LayerNorm

    x = torch.randn(4, 64)
    with need_xpu_graph_logs():
        got = torch.compile(fn, backend=backend)(x)
    torch.testing.assert_close(got, fn(x))
    assert "Pattern.FusedLayerNorm changed graph" not in caplog.text


def test_level1_leaves_norms_alone(caplog):
    be = XpuGraph(XpuGraphConfig(is_training=False))  # the default path: level1, target none
    x, w = torch.randn(8, 64), torch.randn(64)
    with need_xpu_graph_logs():
        got = torch.compile(rms_baseline_c1, backend=be)(x, w)
    assert torch.equal(got, rms_baseline_c1(x, w))  # level1 is bitwise-preserving
    assert "FusedRMSNorm" not in caplog.text.replace("skip", "")
